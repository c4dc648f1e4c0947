// The quantised product for a pass of at most 16 rows through a SMALL model (the drafter's passes
// of the tree loop: 8 rows, layers of a few MB, where every launch is launch latency and the
// number of dependent launches per layer is what counts), with the operators around the product
// folded in so that a decoder layer needs four of these launches and no norm / add launch:
//
//   out = (RMSNorm(x, norm_w) or x) . W^T  (+ bias)              q|k|v
//   out = residual + fp16(x . W^T)                               o and down projections, in place on h
//   out = silu(g) * u,  (g | u) = (RMSNorm(x) or x) . Wgu^T      gate|up, interleaved 16-row tiles
//
// (mlx_llama.py:195-196, 214-215, 225-249).
//
//   * A workgroup owns one 16-row weight tile (a (gate, up) pair for SwiGLU); its four or eight
//     waves deal the 128-column chunks of K among themselves (one to five each) and add their
//     tiles in LDS.  Every request of a wave (weights, scales, its columns of x as the B operand
//     of v_mfma_f32_16x16x32_f16) is in flight together; there is no loop over K, and the chain
//     of dependent instructions per wave is a few hundred long.  (One wave per tile over the whole
//     K was measured first: 2500 dependent instructions on one wave per SIMD, 15 us per launch.)
//   * The norm is folded into the load of x: each wave sums the squares of its columns, the row
//     sums are added across the waves in LDS; no launch and no pass over memory for it.
//   * Expansion of the nibbles through fp16 subnormals as in csrc/resident.hip: fp16(s q + b),
//     single rounding; scales below 0.2499.
//
// A form of this file that ran a whole layer as ONE resident grid with grid-wide barriers between
// the products was measured and dropped: a barrier plus the first load behind it costs what a
// launch costs (56 us per layer against 33 us for the launches it replaced).
#include "common.h"

namespace {

typedef __attribute__((address_space(3))) float4_t sp_lds_float4;

__device__ inline half8_t sp_permute8(half8_t v) {
  return half8_t{v[0], v[4], v[1], v[5], v[2], v[6], v[3], v[7]};
}

// eight nibbles -> fp16(s q + b), in the order q0 q4 q1 q5 q2 q6 q3 q7
__device__ inline half8_t sp_dequant(uint32_t w, half2_t s18, half2_t b2) {
  union { uint32_t u; half2_t h; } c[4];
  c[0].u = (w << 6) & 0x03c003c0u;
  c[1].u = (w << 2) & 0x03c003c0u;
  c[2].u = (w >> 2) & 0x03c003c0u;
  c[3].u = (w >> 6) & 0x03c003c0u;
  half8_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t v = __builtin_elementwise_fma(c[i].h, s18, b2);
    o[2 * i] = v[0];
    o[2 * i + 1] = v[1];
  }
  return o;
}

struct SmallArgs {
  const half_t* x;          // [T, K]
  const half_t* norm_w;     // [K] or nullptr
  const uint32_t* w;        // [N, K / 8]
  const half_t* s;          // [N, K / 64]
  const half_t* b;
  const half_t* bias;       // [N] or nullptr
  const half_t* residual;   // [T, N] or nullptr
  half_t* out;              // [T, N] ([T, N / 2] for SwiGLU)
  float eps;
  int T, N, K;
};

// NW waves per workgroup, at most MAXC chunks of 128 columns per wave, NT tiles per workgroup
// (2: a (gate, up) pair with the SwiGLU epilogue).  Lane (r = lane % 16, kq = lane / 16) of a
// wave holds, per chunk, weight row r columns 32 kq .. + 32 (one 16-byte load, four packed words,
// one per matrix instruction) and x row r at the same columns; the accumulator of lane (m, q4)
// is weight rows 4 q4 .. + 4 of x row m.
template <int NW, int MAXC, int NT>
__global__ __launch_bounds__(NW * 64) void qmm_small_kernel(SmallArgs a) {
  __shared__ __attribute__((aligned(16))) float4_t red[NW][NT][64];
  __shared__ float ssq[NW][16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, kq = lane >> 4;
  const int K = a.K, KW = K >> 3, G = K >> 6;
  // chunks dealt over the waves as evenly as they go
  const int chunks = K >> 7;
  const int per = chunks / NW, rem = chunks % NW;
  const int nch = per + (wave < rem ? 1 : 0);
  const int k0 = (wave * per + (wave < rem ? wave : rem)) * 128;
  const int row0 = blockIdx.x * (16 * NT);

  // ---- every request of the wave at once ----
  uint4_t wv[NT][MAXC];
  half_t sv[NT][MAXC], bv[NT][MAXC];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const long row = row0 + 16 * t + r;
    const uint32_t* wp = a.w + row * KW + (k0 >> 3) + kq * 4;
    const half_t* sp = a.s + row * G + (k0 >> 6) + (kq >> 1);
    const half_t* bp = a.b + row * G + (k0 >> 6) + (kq >> 1);
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nch) {
        wv[t][c] = *reinterpret_cast<const uint4_t*>(wp + c * 16);
        sv[t][c] = sp[c * 2];
        bv[t][c] = bp[c * 2];
      }
    }
  }
  half8_t xb[MAXC][4];
  const bool live = r < a.T;
  const half_t* xp = a.x + (long)(live ? r : 0) * K + k0 + kq * 32;
#pragma unroll
  for (int c = 0; c < MAXC; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      xb[c][i] = (c < nch && live) ? *reinterpret_cast<const half8_t*>(xp + c * 128 + i * 8)
                                   : half8_t{0, 0, 0, 0, 0, 0, 0, 0};

  // ---- RMSNorm folded into x ----
  if (a.norm_w) {
    half8_t nw[MAXC][4];
    const half_t* np = a.norm_w + k0 + kq * 32;
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (c < nch) nw[c][i] = *reinterpret_cast<const half8_t*>(np + c * 128 + i * 8);
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += (float)xb[c][i][e] * (float)xb[c][i][e];
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (kq == 0) ssq[wave][r] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) tot += ssq[w][r];
    const float rinv = 1.0f / sqrtf(tot / (float)K + a.eps);
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nch) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          half8_t o;
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)nw[c][i][e] * ((float)xb[c][i][e] * rinv));
          xb[c][i] = o;
        }
      }
    }
  }

  // ---- the wave's part of the tile(s) ----
  float4_t acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nch) {
        const half_t sc = (half_t)((float)sv[t][c] * 262144.f);
        const half_t bi = bv[t][c];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const half8_t av = sp_dequant(wv[t][c][i], half2_t{sc, sc}, half2_t{bi, bi});
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, sp_permute8(xb[c][i]), acc[t], 0, 0, 0);
        }
      }
    }
    *(sp_lds_float4*)&red[wave][t][lane] = acc[t];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    float4_t sum = red[0][t][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[w][t][lane];
    acc[t] = sum;
  }

  // ---- epilogue: lane (m, q4) holds weight rows row0 (+ 16) + 4 q4 .. + 4 of x row m ----
  const int m = r, q4 = kq;
  if (m >= a.T) return;
  if (NT == 2) {
    const int n_g = row0 + 4 * q4;                      // gate rows; the matching up rows are 16 further
    half4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half_t g = (half_t)acc[0][i], u = (half_t)acc[NT - 1][i];
      if (a.bias) {
        g = g + a.bias[n_g + i];
        u = u + a.bias[n_g + 16 + i];
      }
      const float gf = (float)g;
      const half_t act = (half_t)(gf / (1.0f + expf(-gf)));
      o[i] = (half_t)((float)act * (float)u);
    }
    *reinterpret_cast<half4_t*>(a.out + (long)m * (a.N >> 1) + (row0 >> 1) + 4 * q4) = o;
  } else {
    const int n = row0 + 4 * q4;
    half4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = (half_t)acc[0][i];
      if (a.bias) o[i] = o[i] + a.bias[n + i];
    }
    if (a.residual) {
      const half4_t res = *reinterpret_cast<const half4_t*>(a.residual + (long)m * a.N + n);
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (half_t)((float)o[i] + (float)res[i]);
    }
    *reinterpret_cast<half4_t*>(a.out + (long)m * a.N + n) = o;
  }
}

constexpr int SMALL_K4 = 4 * 3 * 128;      // four waves, three chunks each
constexpr int SMALL_K8 = 8 * 5 * 128;      // eight waves, five chunks each

}  // namespace

EAGLE_EXPORT int eagle_qmm_small_supported(int T, int N, int K, int norm, int swiglu) {
  (void)norm;
  return T >= 1 && T <= 16 && N >= 16 && (N % (swiglu ? 32 : 16)) == 0 && K >= 128 && (K % 128) == 0 &&
         K <= SMALL_K8;
}

EAGLE_EXPORT int eagle_qmm_small_w4g64_f16(const void* x, const void* norm_w, float eps, const uint32_t* wq,
                                           const void* scales, const void* biases, const void* bias,
                                           const void* residual, void* out, int T, int N, int K,
                                           int group_size, int bits, int swiglu, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (!eagle_qmm_small_supported(T, N, K, norm_w != nullptr, swiglu)) return EAGLE_ERR_SHAPE;
  if (swiglu && residual) return EAGLE_ERR_UNSUPPORTED;
  const void* aligned[] = {x, norm_w, wq, residual, out};
  for (const void* p : aligned)
    if (p && !eagle_aligned16(p)) return EAGLE_ERR_ALIGN;
  if (x == out) return EAGLE_ERR_UNSUPPORTED;          // other workgroups still read x
  SmallArgs a;
  a.x = static_cast<const half_t*>(x);
  a.norm_w = static_cast<const half_t*>(norm_w);
  a.w = wq;
  a.s = static_cast<const half_t*>(scales);
  a.b = static_cast<const half_t*>(biases);
  a.bias = static_cast<const half_t*>(bias);
  a.residual = static_cast<const half_t*>(residual);
  a.out = static_cast<half_t*>(out);
  a.eps = eps;
  a.T = T;
  a.N = N;
  a.K = K;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool wide = K > SMALL_K4;
  if (swiglu) {
    if (wide)
      hipLaunchKernelGGL((qmm_small_kernel<8, 5, 2>), dim3(N / 32), dim3(512), 0, st, a);
    else
      hipLaunchKernelGGL((qmm_small_kernel<4, 3, 2>), dim3(N / 32), dim3(256), 0, st, a);
  } else {
    if (wide)
      hipLaunchKernelGGL((qmm_small_kernel<8, 5, 1>), dim3(N / 16), dim3(512), 0, st, a);
    else
      hipLaunchKernelGGL((qmm_small_kernel<4, 3, 1>), dim3(N / 16), dim3(256), 0, st, a);
  }
  return eagle_launch_status();
}
