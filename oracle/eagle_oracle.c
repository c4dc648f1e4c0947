/*
 * CPU restatement of the EAGLE-2 tree-verification operators.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared
 * against (tests, the smoke check and the cpu_baseline leg of the benchmark).
 * Nothing in the shipped package may call into it.
 *
 * Every tensor of half-precision data is passed as raw IEEE binary16 bit
 * patterns (uint16_t).  All arithmetic is fp32 (or wider), with one rounding
 * to fp16 where the reference graph materialises an fp16 tensor.
 *
 * Parity pins (see tests/test_oracle_*.py):
 *   orc_qmm_w4g64       float64 closed form, one-hot/known-answer cases,
 *                       integer-exact case, torch.matmul on dequantised weights
 *   orc_rope_arrayed    float64 closed form, permutation invariant of the
 *                       reference self-check, transformers rotate_half form
 *   orc_tree_attention  torch SDPA with additive mask + GQA, path invariant
 *   orc_rmsnorm/silu    textbook closed forms (torch)
 *   orc_embed_w4g64     one-hot QMM identity
 *   orc_argmax_rows     numpy argmax (first maximum)
 * The exact fp16 bit patterns of the MLX CPU kernels (accumulation order,
 * sin/cos implementation) are "parity unpinned": MLX is not available; the
 * tolerance max|err| <= 2e-2 * RMS(out) covers them.
 *
 * Build: see oracle/Makefile (gcc -O3 -mavx2 -mfma -mf16c -fopenmp).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

static inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }

ORC_API void orc_h2f(const uint16_t* in, float* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = h2f(in[i]);
}
ORC_API void orc_f2h(const float* in, uint16_t* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = f2h(in[i]);
}

/*
 * 4-bit affine quantised matmul, group size 64.
 *   out[m,n] = fp16( sum_k x[m,k] * (s[n,k/64] * q[n,k] + b[n,k/64]) )  (+ bias[n])
 *   q[n,k]   = (w[n,k/8] >> 4*(k%8)) & 15
 * Layout and nibble order: reference kernels/progression/simd_no_swizzle_cast.metal:52-53,82-125
 * and kernels/qmv/1.metal:26-51; call contract qmm_kernel.py:84-164.
 * fp32 accumulation, one fp16 rounding of the result.  The optional bias is
 * added to the rounded result in fp16, as the patched linear layer does after
 * the kernel returns (mlx_model_fwd_bench.py:69-71).
 */
/* Weight rounding of orc_qmm_w4g64: 0 (default) keeps s*q + b in fp32; 1 rounds every
 * dequantised weight to fp16 first, as the reference Metal kernel holds them (half2
 * `w1 = w1 * s0 + b0`, kernels/progression/simd_no_swizzle_cast.metal:82-84).  Both are the
 * reference's arithmetic (MLX CPU path and Metal path); tests use 1 to separate the rounding of
 * the weights from other differences.  Pinned by the same float64 closed form with the
 * weights rounded. */
static int orc_round_weights = 0;
ORC_API void orc_set_weight_rounding(int on) { orc_round_weights = on ? 1 : 0; }

ORC_API int orc_qmm_w4g64(const uint16_t* x, const uint32_t* w, const uint16_t* s,
                          const uint16_t* b, const uint16_t* bias, uint16_t* out,
                          int M, int N, int K) {
  if (M < 1 || N < 1 || K < 64 || (K % 64) != 0) return 1;
  const int G = K / 64;
  float* xf = (float*)malloc((size_t)M * K * sizeof(float));
  if (!xf) return 2;
  for (long i = 0; i < (long)M * K; ++i) xf[i] = h2f(x[i]);
#pragma omp parallel
  {
    float* wf = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
    for (int n = 0; n < N; ++n) {
      const uint32_t* wr = w + (size_t)n * (K / 8);
      for (int g = 0; g < G; ++g) {
        const float sc = h2f(s[(size_t)n * G + g]);
        const float bi = h2f(b[(size_t)n * G + g]);
        for (int j = 0; j < 8; ++j) {
          const uint32_t word = wr[g * 8 + j];
          for (int i = 0; i < 8; ++i)
            wf[g * 64 + j * 8 + i] = sc * (float)((word >> (4 * i)) & 15u) + bi;
        }
      }
      if (orc_round_weights)
        for (int k = 0; k < K; ++k) wf[k] = h2f(f2h(wf[k]));
      for (int m = 0; m < M; ++m) {
        const float* xr = xf + (size_t)m * K;
        float acc = 0.f;
#pragma omp simd reduction(+ : acc)
        for (int k = 0; k < K; ++k) acc += xr[k] * wf[k];
        uint16_t r = f2h(acc);
        if (bias) r = f2h(h2f(r) + h2f(bias[n]));
        out[(size_t)m * N + n] = r;
      }
    }
    free(wf);
  }
  free(xf);
  return 0;
}

/*
 * Quantised-embedding gather: out[t,:] = fp16(s*q + b) for row ids[t].
 * (mlx_llama.py:273; the embedding is quantised like every linear layer,
 * mlx_utils.py:123-134.)
 */
ORC_API int orc_embed_w4g64(const int32_t* ids, const uint32_t* w, const uint16_t* s,
                            const uint16_t* b, uint16_t* out, int T, int D, int V) {
  if ((D % 64) != 0) return 1;
  const int G = D / 64;
  for (int t = 0; t < T; ++t) {
    const int id = ids[t];
    if (id < 0 || id >= V) return 3;
    for (int k = 0; k < D; ++k) {
      const uint32_t word = w[(size_t)id * (D / 8) + k / 8];
      const float q = (float)((word >> (4 * (k % 8))) & 15u);
      const float sc = h2f(s[(size_t)id * G + k / 64]);
      const float bi = h2f(b[(size_t)id * G + k / 64]);
      out[(size_t)t * D + k] = f2h(fmaf(sc, q, bi));
    }
  }
  return 0;
}

/*
 * RoPE with one integer position per (batch, token), half-split pairing.
 *   theta = (scale * inv_freq[i]) * (float)pos[b,t]           (fp32 products)
 *   o[i]      = x[i] cos(theta) - x[i+hd/2] sin(theta)
 *   o[i+hd/2] = x[i] sin(theta) + x[i+hd/2] cos(theta)
 * x, out: contiguous [B,H,L,hd] fp16.  Reference: mlx_arrayed_rope_kernel.py:60-123
 * (theta :66-68,:98-99; rotation :105-117; pairing :81-86).
 */
ORC_API int orc_rope_arrayed(const uint16_t* x, const int32_t* pos, const float* inv_freq,
                             float scale, uint16_t* out, int B, int H, int L, int hd) {
  if (hd % 2) return 1;
  const int half = hd / 2;
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
      for (int t = 0; t < L; ++t) {
        const size_t base = (((size_t)b * H + h) * L + t) * hd;
        const float p = (float)pos[(size_t)b * L + t];
        for (int i = 0; i < half; ++i) {
          const float lf = scale * inv_freq[i];
          const float theta = lf * p;
          const float c = (float)cos((double)theta);
          const float sn = (float)sin((double)theta);
          const float x1 = h2f(x[base + i]);
          const float x2 = h2f(x[base + i + half]);
          out[base + i] = f2h(x1 * c - x2 * sn);
          out[base + i + half] = f2h(x1 * sn + x2 * c);
        }
      }
  return 0;
}

/*
 * softmax(scale * Q K^T + mask) V with grouped-query heads.
 *   q    [H, T, hd]           fp16
 *   k, v [G, kv_stride, hd]   fp16, first S rows of each head are used
 *   mask [T, S]               fp16 additive ({0, -inf} on the tree path)
 *   out  [H, T, hd]           fp16
 * q head h reads kv head h / (H/G).  Scores, softmax and the weighted sum are
 * fp32.  Call site: mlx_llama.py:185-192; mask construction mlx_eagle.py:337-338.
 */
ORC_API int orc_tree_attention(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                               const uint16_t* mask, uint16_t* out, int H, int G, int T,
                               int S, int hd, long kv_stride, float scale) {
  if (H % G) return 1;
  const int rep = H / G;
#pragma omp parallel for collapse(2) schedule(static)
  for (int h = 0; h < H; ++h)
    for (int t = 0; t < T; ++t) {
      const int g = h / rep;
      float* sc = (float*)malloc((size_t)S * sizeof(float));
      float* acc = (float*)calloc((size_t)hd, sizeof(float));
      const uint16_t* qr = q + ((size_t)h * T + t) * hd;
      float mx = -INFINITY;
      for (int j = 0; j < S; ++j) {
        const uint16_t* kr = k + ((size_t)g * kv_stride + j) * hd;
        float d = 0.f;
        for (int e = 0; e < hd; ++e) d += h2f(qr[e]) * h2f(kr[e]);
        d = d * scale + h2f(mask[(size_t)t * S + j]);
        sc[j] = d;
        if (d > mx) mx = d;
      }
      float den = 0.f;
      for (int j = 0; j < S; ++j) {
        const float p = (sc[j] == -INFINITY) ? 0.f : expf(sc[j] - mx);
        sc[j] = p;
        den += p;
      }
      for (int j = 0; j < S; ++j) {
        if (sc[j] == 0.f) continue;
        const uint16_t* vr = v + ((size_t)g * kv_stride + j) * hd;
        for (int e = 0; e < hd; ++e) acc[e] += sc[j] * h2f(vr[e]);
      }
      uint16_t* o = out + ((size_t)h * T + t) * hd;
      for (int e = 0; e < hd; ++e) o[e] = f2h(acc[e] / den);
      free(sc);
      free(acc);
    }
  return 0;
}

/* RMSNorm, fp32 math, fp16 in/out: out = w * x * rsqrt(mean(x^2) + eps).  mlx_llama.py:225-228,240,247,286. */
ORC_API void orc_rmsnorm(const uint16_t* x, const uint16_t* w, float eps, uint16_t* out,
                         int T, int D) {
  for (int t = 0; t < T; ++t) {
    double ss = 0.0;
    for (int d = 0; d < D; ++d) {
      const float v = h2f(x[(size_t)t * D + d]);
      ss += (double)v * v;
    }
    const float r = 1.0f / sqrtf((float)(ss / D) + eps);
    for (int d = 0; d < D; ++d)
      out[(size_t)t * D + d] = f2h(h2f(w[d]) * (h2f(x[(size_t)t * D + d]) * r));
  }
}

/* out = fp16( fp16(silu(g)) * u ), silu(g) = g / (1 + exp(-g)).  mlx_llama.py:215. */
ORC_API void orc_silu_mul(const uint16_t* g, const uint16_t* u, uint16_t* out, long n) {
  for (long i = 0; i < n; ++i) {
    const float gv = h2f(g[i]);
    const uint16_t a = f2h(gv / (1.0f + expf(-gv)));
    out[i] = f2h(h2f(a) * h2f(u[i]));
  }
}

/* out = fp16(a + b): the residual adds of mlx_llama.py:246,248. */
ORC_API void orc_add(const uint16_t* a, const uint16_t* b, uint16_t* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = f2h(h2f(a[i]) + h2f(b[i]));
}

/* Row argmax of fp16 logits, lowest index among equal maxima (mlx_eagle.py:316,534,596). */
ORC_API void orc_argmax_rows(const uint16_t* logits, int32_t* out, int R, long V) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < R; ++r) {
    const uint16_t* row = logits + (size_t)r * V;
    float best = h2f(row[0]);
    long bi = 0;
    for (long j = 1; j < V; ++j) {
      const float val = h2f(row[j]);
      if (val > best) {
        best = val;
        bi = j;
      }
    }
    out[r] = (int32_t)bi;
  }
}
