// The quantised product for a pass of at most 16 rows through a SMALL model (the drafter's passes
// of the tree loop: 8 rows, layers of a few MB, where every launch is launch latency and the
// number of dependent launches per layer is what counts), with the operators around the product
// folded in so that a decoder layer needs four of these launches and no norm / add launch:
//
//   out = (RMSNorm(x, norm_w) or x) . W^T  (+ bias)              q|k|v
//   out = residual + fp16(x . W^T)                               o and down projections, in place on h
//   out = silu(g) * u,  (g | u) = (RMSNorm(x) or x) . Wgu^T      gate|up, interleaved 16-row tiles
//   q [H,T,hd], cache rows = rope(RMSNorm(x) . Wqkv^T + bias)    q|k|v with rotation and cache append
//
// (mlx_llama.py:195-196, 214-215, 225-249).
//
//   * A workgroup owns one 16-row weight tile (a (gate, up) pair for SwiGLU, the two halves of a
//     head that a rotation pairs for rope); its four, eight or sixteen waves deal the 128-column
//     chunks of K among themselves (at most three each) and add their tiles in LDS.  Every request
//     of a wave (weights, scales, its columns of x as the B operand of v_mfma_f32_16x16x32_f16) is
//     in flight together; there is no loop over K.
//   * The norm is folded into the load of x: each wave sums the squares of its columns, the row
//     sums are added across the waves in LDS; no launch and no pass over memory for it.  Every
//     workgroup repeats it, so it is kept short: v_dot2 for the sums, x / rms rounded to fp16 and
//     then multiplied by the norm weight in packed fp16 (two roundings where the norm launch has
//     one).
//   * Expansion of the nibbles through fp16 subnormals (a masked nibble pair at mantissa bits
//     6..9 is q * 2^-18 exactly; one packed fma with (s * 2^18, b)): fp16(s q + b), single
//     rounding; scales below 0.2499.
//
// Measured on the way (8 rows, the 0.5B drafter's shapes, launches back to back in a graph):
//   - one wave per tile over the whole K: 2500 instructions on one wave per SIMD, 15 us per launch;
//   - K over the waves, loads under conditions (zero for what a wave does not own): the requests
//     of a wave wait for one another where the branches join; time grows by 1.1 us per chunk;
//   - unconditional loads, 16 bytes per lane straight into the operand layout: the time follows
//     the number of cache lines the load instructions of a compute unit touch (x: 64 per chunk,
//     scales 16 per 2-byte load), 7.8 us for the down projection; shaped as below: 5.7 us;
//   - a whole layer as ONE resident grid with grid-wide barriers between the products: a barrier
//     plus the first load behind it costs what a launch costs (56 us per layer against 33 us for
//     the launches it replaced);
//   - attention of such a pass in one launch (a workgroup per query head, keys over its sixteen
//     waves, merge through LDS): 14.7 to 30.8 us against 9.9 to 13.4 us for the split and merge
//     launches over 64 to 2048 keys.
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
  // rope form: (cos, sin) table [T, hd / 2, 2], rotated q [H, T, hd], caches [G, cap, hd], *len_dev = row of
  // the first new K / V row
  const float* rope_cs;
  half_t* q_out;
  half_t* k_cache;
  half_t* v_cache;
  const int32_t* len_dev;
  int H, G, hd;
  long cap;
};

enum { SMALL_PLAIN = 0, SMALL_SWIGLU = 1, SMALL_ROPE = 2 };

// NW waves per workgroup, at most SMALL_MAXC chunks of 128 columns per wave, RP passes of four x rows
// (2: T <= 8, 4: T <= 16).  MODE: one tile per workgroup (plain / residual), a (gate, up) tile pair
// 16 rows apart with the SwiGLU epilogue, or two tiles of one head half a head apart (the two
// halves a rotation pairs) with the rope epilogue.  Lane (r = lane % 16, kq = lane / 16) of a wave
// holds, per chunk, weight row r columns 32 kq .. + 32 (one 16-byte load, four packed words, one
// per matrix instruction) and x row r at the same columns; the accumulator of lane (m, q4) is
// weight rows 4 q4 .. + 4 of x row m.
//
// What bounds this kernel is the number of cache lines its load instructions touch per compute
// unit, so every request is shaped for few lines: x is read with whole rows of a chunk per
// instruction (four rows x 256 bytes) and brought into the operand layout through a per-wave LDS
// buffer; the two scales (biases) of a chunk come as one 4-byte load for the three chunks of a
// wave at once and are handed to the lanes that need them with a lane shuffle.
constexpr int SMALL_MAXC = 3;
constexpr int SMALL_XROW = 256 + 16;       // bytes per staged x row: 128 columns, padded against bank conflicts

template <int NW, int RP, int MODE, bool NORM>
__global__ __launch_bounds__(NW * 64) void qmm_small_kernel(SmallArgs a) {
  constexpr int NT = MODE == SMALL_PLAIN ? 1 : 2;
  constexpr int MAXC = SMALL_MAXC;
  __shared__ __attribute__((aligned(16))) float4_t red[NW][NT][64];
  __shared__ __attribute__((aligned(16))) unsigned char xstage[NW][RP * 4 * SMALL_XROW];
  __shared__ float ssq[NW][16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, kq = lane >> 4;
  const int K = a.K, KW = K >> 3, G = K >> 6;
  // chunks dealt over the waves as evenly as they go
  const int chunks = K >> 7;
  const int per = chunks / NW, rem = chunks % NW;
  const int nch = per + (wave < rem ? 1 : 0);
  const int k0 = (wave * per + (wave < rem ? wave : rem)) * 128;
  int row0, second;                       // first row of tile 0, distance of tile 1
  if (MODE == SMALL_ROPE) {
    const int per_head = a.hd >> 5;
    row0 = (blockIdx.x / per_head) * a.hd + (blockIdx.x % per_head) * 16;
    second = a.hd >> 1;
  } else {
    row0 = blockIdx.x * (16 * NT);
    second = 16;
  }

  // ---- every request of the wave at once ----
  // All loads are unconditional (a load under a condition has to be waited for where the branches
  // join, which puts the requests of a wave one behind the other): chunks the wave does not own
  // and rows past T read a valid address again and their values are never used.
  const int kb = nch > 0 ? k0 : 0;
  uint4_t wv[NT][MAXC];
  uint32_t spair[NT], bpair[NT];          // lane (r, c): the two scales (biases) of row r in chunk c
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const long row = row0 + second * t + r;
    const uint32_t* wp = a.w + row * KW + (kb >> 3) + kq * 4;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) wv[t][c] = *reinterpret_cast<const uint4_t*>(wp + (c < nch ? c : 0) * 16);
    const int cpair = kq < nch ? kq : 0;
    spair[t] = *reinterpret_cast<const uint32_t*>(a.s + row * G + (kb >> 6) + cpair * 2);
    bpair[t] = *reinterpret_cast<const uint32_t*>(a.b + row * G + (kb >> 6) + cpair * 2);
  }
  // x: lane l reads 16 bytes of row 4 p + l / 16 at byte 16 (l % 16) of the chunk's 256
  uint4_t xg[MAXC][RP];
  {
    const int xr = lane >> 4, xc = lane & 15;
#pragma unroll
    for (int p = 0; p < RP; ++p) {
      int row = 4 * p + xr;
      row = row < a.T ? row : a.T - 1;
      const half_t* xp = a.x + (long)row * K + kb + xc * 8;
#pragma unroll
      for (int c = 0; c < MAXC; ++c) xg[c][p] = *reinterpret_cast<const uint4_t*>(xp + (c < nch ? c : 0) * 128);
    }
  }
  half8_t nw[MAXC][4];
  if (NORM && a.norm_w) {
    const half_t* np = a.norm_w + kb + kq * 32;
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) nw[c][i] = *reinterpret_cast<const half8_t*>(np + (c < nch ? c : 0) * 128 + i * 8);
  }
  // what the epilogue of wave 0 adds (bias, residual, the rotation's cos / sin, the cache length)
  // is requested here with everything else, not after the product: a load behind the product is
  // a microsecond of latency on the critical path of a kernel that takes four.  The values are
  // only read under the conditions they were loaded under.
  half4_t e_bias0, e_bias1, e_res;
  float4_t e_cs[2];
  long e_len = 0;
  const int e_rope_head = MODE == SMALL_ROPE ? row0 / a.hd : 0;
  if (wave == 0) {
    const int bn = row0 + 4 * kq;
    if (a.bias) {
      e_bias0 = *reinterpret_cast<const half4_t*>(a.bias + bn);
      if (NT == 2) e_bias1 = *reinterpret_cast<const half4_t*>(a.bias + bn + second);
    }
    if (MODE == SMALL_PLAIN && a.residual && r < a.T)
      e_res = *reinterpret_cast<const half4_t*>(a.residual + (long)r * a.N + bn);
    if (MODE == SMALL_ROPE) {
      e_len = *a.len_dev;
      if (r < a.T && e_rope_head < a.H + a.G) {
        const int d = row0 - e_rope_head * a.hd + 4 * kq;
        const float4_t* cs = reinterpret_cast<const float4_t*>(a.rope_cs + ((long)r * (a.hd >> 1) + d) * 2);
        e_cs[0] = cs[0];
        e_cs[1] = cs[1];
      }
    }
  }
  // x through the wave's LDS buffer into the operand layout, a chunk at a time (rows past 4 RP,
  // which are rows past T, read what is there: their columns of the result are not stored)
  half8_t xb[MAXC][4];
  {
    unsigned char* xs = xstage[wave];
    const int xr = lane >> 4, xc = lane & 15;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
#pragma unroll
      for (int p = 0; p < RP; ++p)
        *reinterpret_cast<uint4_t*>(xs + (4 * p + xr) * SMALL_XROW + xc * 16) = xg[c][p];
      __builtin_amdgcn_wave_barrier();
      const int mr = r < 4 * RP ? r : 0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xb[c][i] = *reinterpret_cast<const half8_t*>(xs + mr * SMALL_XROW + (4 * kq + i) * 16);
      __builtin_amdgcn_wave_barrier();
    }
  }

  // ---- RMSNorm folded into x ----
  if (NORM && a.norm_w) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nch) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const half2_t p2 = half2_t{xb[c][i][e], xb[c][i][e + 1]};
            ss = __builtin_amdgcn_fdot2(p2, p2, ss, false);      // exact products, fp32 sum
          }
      }
    }
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
          for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)xb[c][i][e] * rinv);   // fp32 product, one rounding
          xb[c][i] = o * nw[c][i];                                                      // packed fp16 products
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
        // the pair of chunk c sits in lane (r, c); this lane's columns are in its half kq / 2
        const uint32_t s2 = __shfl(spair[t], r + 16 * c, 64), b2 = __shfl(bpair[t], r + 16 * c, 64);
        const half_t sraw = __builtin_bit_cast(half_t, (unsigned short)(kq & 2 ? s2 >> 16 : s2 & 0xffffu));
        const half_t bi = __builtin_bit_cast(half_t, (unsigned short)(kq & 2 ? b2 >> 16 : b2 & 0xffffu));
        const half_t sc = (half_t)((float)sraw * 262144.f);
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
  if (MODE == SMALL_ROPE) {
    // the linear output rounded to fp16 (bias added in fp16), rotated with the table's (cos, sin)
    // exactly as the separate rope launch does; v rows pass through
    const int half = a.hd >> 1;
    const int hb = e_rope_head;
    const int d = row0 - hb * a.hd + 4 * q4;            // < hd / 2
    half4_t lo, hi;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[i] = (half_t)acc[0][i];
      hi[i] = (half_t)acc[NT - 1][i];
      if (a.bias) {
        lo[i] = lo[i] + e_bias0[i];
        hi[i] = hi[i] + e_bias1[i];
      }
    }
    const long P = e_len;
    if (P + m >= a.cap) return;                         // the host checks capacity; never write past the buffer
    half_t* dst;
    if (hb < a.H) {
      dst = a.q_out + ((long)hb * a.T + m) * a.hd;
    } else {
      const int g = hb < a.H + a.G ? hb - a.H : hb - a.H - a.G;
      dst = (hb < a.H + a.G ? a.k_cache : a.v_cache) + ((long)g * a.cap + P + m) * a.hd;
    }
    if (hb < a.H + a.G) {
      half4_t olo, ohi;
#pragma unroll
      for (int j2 = 0; j2 < 2; ++j2) {
        const float4_t v = e_cs[j2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int j = 2 * j2 + e;
          const float co = v[2 * e], sn = v[2 * e + 1];
          const float x1 = (float)lo[j], x2 = (float)hi[j];
          olo[j] = (half_t)__builtin_fmaf(x1, co, -(x2 * sn));
          ohi[j] = (half_t)__builtin_fmaf(x1, sn, x2 * co);
        }
      }
      lo = olo;
      hi = ohi;
    }
    *reinterpret_cast<half4_t*>(dst + d) = lo;
    *reinterpret_cast<half4_t*>(dst + half + d) = hi;
  } else if (MODE == SMALL_SWIGLU) {
    const int n_g = row0 + 4 * q4;                      // gate rows; the matching up rows are 16 further
    half4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half_t g = (half_t)acc[0][i], u = (half_t)acc[NT - 1][i];
      if (a.bias) {
        g = g + e_bias0[i];
        u = u + e_bias1[i];
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
      if (a.bias) o[i] = o[i] + e_bias0[i];
    }
    if (a.residual) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (half_t)((float)o[i] + (float)e_res[i]);
    }
    *reinterpret_cast<half4_t*>(a.out + (long)m * a.N + n) = o;
  }
}

constexpr int SMALL_K4 = 4 * SMALL_MAXC * 128;       // four waves, three chunks each
constexpr int SMALL_K8 = 8 * SMALL_MAXC * 128;
constexpr int SMALL_K16 = 16 * SMALL_MAXC * 128;

template <int MODE>
void small_launch(const SmallArgs& a, int grid, hipStream_t st) {
  const bool tall = a.T > 8;
#define SMALL_GO(NW, NORM)                                                                                \
  do {                                                                                                 \
    if (tall)                                                                                          \
      hipLaunchKernelGGL((qmm_small_kernel<NW, 4, MODE, NORM>), dim3(grid), dim3(NW * 64), 0, st, a);  \
    else                                                                                               \
      hipLaunchKernelGGL((qmm_small_kernel<NW, 2, MODE, NORM>), dim3(grid), dim3(NW * 64), 0, st, a);  \
  } while (0)
  // Sixteen waves leave a wave 128 registers: the norm weights of its chunks (48 of them) only
  // have room in a build of their own, so the products without a norm (o, down) get one that
  // does not hold them.
  if (a.K <= SMALL_K4)
    SMALL_GO(4, true);
  else if (a.K <= SMALL_K8)
    SMALL_GO(8, true);
  else if (a.norm_w)
    SMALL_GO(16, true);
  else
    SMALL_GO(16, false);
#undef SMALL_GO
}

}  // namespace

EAGLE_EXPORT int eagle_qmm_small_supported(int T, int N, int K, int norm, int swiglu) {
  (void)norm;
  return T >= 1 && T <= 16 && N >= 16 && (N % (swiglu ? 32 : 16)) == 0 && K >= 128 && (K % 128) == 0 &&
         K <= SMALL_K16;
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
  a.rope_cs = nullptr;
  a.q_out = a.k_cache = a.v_cache = nullptr;
  a.len_dev = nullptr;
  a.H = a.G = a.hd = 0;
  a.cap = 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (swiglu)
    small_launch<SMALL_SWIGLU>(a, N / 32, st);
  else
    small_launch<SMALL_PLAIN>(a, N / 16, st);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qkv_rope_small_supported(int T, int D, int H, int G, int hd) {
  return T >= 1 && T <= 16 && H >= 1 && G >= 1 && (H % G) == 0 && hd >= 32 && (hd % 32) == 0 &&
         D >= 128 && (D % 128) == 0 && D <= SMALL_K16;
}

EAGLE_EXPORT int eagle_qkv_rope_small_w4g64_f16(const void* x, const void* norm_w, float eps,
                                                const uint32_t* wq, const void* scales, const void* biases,
                                                const void* bias, const float* rope_cs, void* q_out,
                                                void* k_cache, void* v_cache, const int32_t* cache_len_dev,
                                                int T, int D, int H, int G, int hd, long capacity,
                                                int group_size, int bits, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !rope_cs || !q_out || !k_cache || !v_cache || !cache_len_dev)
    return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (!eagle_qkv_rope_small_supported(T, D, H, G, hd) || capacity < T) return EAGLE_ERR_SHAPE;
  const void* aligned[] = {x, norm_w, wq, rope_cs, q_out, k_cache, v_cache};
  for (const void* p : aligned)
    if (p && !eagle_aligned16(p)) return EAGLE_ERR_ALIGN;
  SmallArgs a;
  a.x = static_cast<const half_t*>(x);
  a.norm_w = static_cast<const half_t*>(norm_w);
  a.w = wq;
  a.s = static_cast<const half_t*>(scales);
  a.b = static_cast<const half_t*>(biases);
  a.bias = static_cast<const half_t*>(bias);
  a.residual = nullptr;
  a.out = nullptr;
  a.eps = eps;
  a.T = T;
  a.N = (H + 2 * G) * hd;
  a.K = D;
  a.rope_cs = rope_cs;
  a.q_out = static_cast<half_t*>(q_out);
  a.k_cache = static_cast<half_t*>(k_cache);
  a.v_cache = static_cast<half_t*>(v_cache);
  a.len_dev = cache_len_dev;
  a.H = H;
  a.G = G;
  a.hd = hd;
  a.cap = capacity;
  hipStream_t st = static_cast<hipStream_t>(stream);
  small_launch<SMALL_ROPE>(a, (H + 2 * G) * (hd / 32), st);
  return eagle_launch_status();
}
