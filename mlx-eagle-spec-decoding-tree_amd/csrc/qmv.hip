// 4-bit group-64 quantised matrix-vector product (one row of x, or a few) on the vector ALU, no
// matrix instructions: out[m][n] = fp16( sum_k x[m][k] (s[n,k/64] q[n,k] + b[n,k/64]) ) (+ bias[n]).
// (Reference: the M = 1 call sites of mx.quantized_matmul, mlx_model_fwd_bench.py:65-73, the
// factorisation of kernels/qmv/1b.metal:121-147: sum q x s + b sum x with a SIMD-group sum, and
// its batched form, kernels/qmv/1b.metal:100-147 with qmv.py:226-241: the expanded weights of a
// packed word are used for every row of the batch.)
//
//   * Sixteen lanes share a weight row: a lane loads 16 bytes (32 weights, half a quantisation
//     group) per step, the sixteen lanes 256 contiguous bytes, a wave four rows at a time; K is
//     walked in steps of 512.  Four steps are in flight per lane.
//   * x sits in LDS as fp16 together with, per 32 columns, the three sums the factorisation needs
//     (all columns, even positions of a packed pair, odd positions); the four row groups of a wave
//     read the same addresses (broadcast).
//   * Nibbles become fp16 by the magic-number trick only ((w & 0x000f000f) | 0x6400 = 1024 + q,
//     (w & 0x00f000f0) | 0x5400 = 64 + 16 q ... see expand below), four v_dot2_f32_f16 per packed
//     word accumulate sum (offset + q) x in fp32; offsets, scale and bias are applied once per
//     lane and step: acc += s (d - 1024 xe - 64 xo) + b xs.
//   * The sixteen partial sums of a row are added with DPP row shifts.
//   * MR rows of x (1, 2, 4 or 8): the expansion of a packed word (one shift, four v_and_or) is
//     shared, the four dot products and the LDS read of x are per row: 5 + 4 MR vector
//     instructions per word.
#include "common.h"

namespace {

constexpr int QMV_WAVES = 4;                 // waves per workgroup
constexpr int QMV_RING = 4;                  // 16-byte loads in flight per lane

__device__ inline uint32_t qmv_and_or(uint32_t v, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(bits));
  return r;
}

__device__ inline float dot2(uint32_t a, half2_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), b, c, false);
}

// sum over the 16 lanes of a DPP row; every lane of the row gets the total
__device__ inline float row_sum16(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));  // row_ror:8
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));  // row_ror:4
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));  // row_ror:2
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));  // row_ror:1
  return v;
}

// LDS: x [K] fp16, then per 32 columns {sum, sum of even pair positions, sum of odd pair
// positions} fp32.  A packed word holds (q0..q7); the expansion below pairs (q0,q4) (q1,q5)
// (q2,q6) (q3,q7): x is stored in that order, "even" = pairs 0 and 2 (offset 1024), "odd" =
// pairs 1 and 3 (offset 64).
template <int MR>
__global__ __launch_bounds__(QMV_WAVES * 64) void qmv_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w, const half_t* __restrict__ s,
    const half_t* __restrict__ b, const half_t* __restrict__ bias, half_t* __restrict__ out, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(16))) unsigned char qmv_lds[];
  half_t* xl = reinterpret_cast<half_t*>(qmv_lds);                       // [MR][K]
  float* corr = reinterpret_cast<float*>(qmv_lds + (size_t)MR * K * 2);   // [MR][K / 32][3]
  const int tid = threadIdx.x;
  const int nthr = QMV_WAVES * 64;
  const int KC = K / 32;
  // stage x: thread t handles words of 8 columns (rows past M repeat the last one; never stored)
  for (int c = tid; c < MR * (K / 8); c += nthr) {
    const int m = c / (K / 8), cc = c % (K / 8);
    const half8_t v = *reinterpret_cast<const half8_t*>(x + (long)(m < M ? m : M - 1) * K + cc * 8);
    *reinterpret_cast<half8_t*>(xl + (long)m * K + cc * 8) = half8_t{v[0], v[4], v[1], v[5], v[2], v[6], v[3], v[7]};
  }
  __syncthreads();
  for (int c = tid; c < MR * KC; c += nthr) {
    const int m = c / KC, cc = c % KC;
    float se = 0.f, so = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const half8_t v = *reinterpret_cast<const half8_t*>(xl + (long)m * K + cc * 32 + j * 8);
      se += (float)v[0] + (float)v[1] + (float)v[4] + (float)v[5];
      so += (float)v[2] + (float)v[3] + (float)v[6] + (float)v[7];
    }
    corr[c * 3] = se + so;
    corr[c * 3 + 1] = se;
    corr[c * 3 + 2] = so;
  }
  __syncthreads();

  const int wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, rg = lane >> 4;
  const int steps = K >> 9;                    // 512 columns per step
  const int G = K >> 6, KW = K >> 3;
  const int rows_per_wg = QMV_WAVES * 4;
  const uint32_t magic_lo = 0x64006400u, magic_hi = 0x54005400u;
  for (long base = (long)blockIdx.x * rows_per_wg; base < N; base += (long)gridDim.x * rows_per_wg) {
    long n = base + wave * 4 + rg;
    const bool live = n < N;
    if (!live) n = N - 1;
    const uint32_t* wp = w + n * KW + l16 * 4;
    const half_t* sp = s + n * G + (l16 >> 1);
    const half_t* bp = b + n * G + (l16 >> 1);
    uint4_t ring[QMV_RING];
    half_t sr[QMV_RING], br[QMV_RING];
#pragma unroll
    for (int r = 0; r < QMV_RING; ++r) {
      const int st = r < steps ? r : steps - 1;
      ring[r] = *reinterpret_cast<const uint4_t*>(wp + st * 64);
      sr[r] = sp[st * 8];
      br[r] = bp[st * 8];
    }
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
    for (int st0 = 0; st0 < steps; st0 += QMV_RING) {
#pragma unroll
      for (int r = 0; r < QMV_RING; ++r) {
        const int st = st0 + r;
        if (st >= steps) break;
        const uint4_t wv = ring[r];
        const float sc = (float)sr[r], bi = (float)br[r];
        const int nx = st + QMV_RING < steps ? st + QMV_RING : steps - 1;
        ring[r] = *reinterpret_cast<const uint4_t*>(wp + nx * 64);
        sr[r] = sp[nx * 8];
        br[r] = bp[nx * 8];
        const int col = st * 512 + l16 * 32;
        float d[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) d[m] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t v = wv[j], v2 = v >> 8;
          // (1024 + q0, 1024 + q4), (64 + q1 .. as 16 q1 in the low mantissa bits of 64: the
          // nibble sits four bits up, so the value is 64 + q), (1024 + q2, 1024 + q6), (64 + q3, 64 + q7)
          const uint32_t e0 = qmv_and_or(v, 0x000f000fu, magic_lo), e1 = qmv_and_or(v, 0x00f000f0u, magic_hi);
          const uint32_t e2 = qmv_and_or(v2, 0x000f000fu, magic_lo), e3 = qmv_and_or(v2, 0x00f000f0u, magic_hi);
#pragma unroll
          for (int m = 0; m < MR; ++m) {
            const half8_t xv = *reinterpret_cast<const half8_t*>(xl + (long)m * K + col + j * 8);
            d[m] = dot2(e0, half2_t{xv[0], xv[1]}, d[m]);
            d[m] = dot2(e1, half2_t{xv[2], xv[3]}, d[m]);
            d[m] = dot2(e2, half2_t{xv[4], xv[5]}, d[m]);
            d[m] = dot2(e3, half2_t{xv[6], xv[7]}, d[m]);
          }
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          const float* cp = corr + ((long)m * KC + (col >> 5)) * 3;
          acc[m] += sc * (d[m] - 1024.f * cp[1] - 64.f * cp[2]) + bi * cp[0];
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float a = row_sum16(acc[m]);
      if (live && l16 == 0 && m < M) {
        half_t o = (half_t)a;
        if (bias) o = o + bias[n];
        out[(long)m * N + n] = o;
      }
    }
  }
}

}  // namespace

static size_t qmv_lds_bytes(int mr, int K) { return (size_t)mr * ((size_t)K * 2 + (size_t)(K / 32) * 12); }

static int qmv_rows_of(int M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : 8; }

EAGLE_EXPORT int eagle_qmv_rows_supported(int M, int N, int K) {
  return M >= 1 && M <= 8 && N >= 8 && K >= 512 && (K % 512) == 0 && qmv_lds_bytes(qmv_rows_of(M), K) <= 150 * 1024;
}

EAGLE_EXPORT int eagle_qmv_supported(int N, int K) { return eagle_qmv_rows_supported(1, N, K); }

template <int MR>
static int qmv_launch(const half_t* x, const uint32_t* wq, const half_t* s, const half_t* b, const half_t* bias,
                      half_t* out, int M, int N, int K, hipStream_t st) {
  const size_t lds = qmv_lds_bytes(MR, K);
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmv_w4g64_kernel<MR>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  const long groups = ((long)N + QMV_WAVES * 4 - 1) / (QMV_WAVES * 4);
  const int per_cu = lds > 48 * 1024 ? 2 : (lds > 24 * 1024 ? 4 : 6);
  const long grid = groups < 256L * per_cu ? groups : 256L * per_cu;
  hipLaunchKernelGGL(qmv_w4g64_kernel<MR>, dim3((unsigned)grid), dim3(QMV_WAVES * 64), lds, st, x, wq, s, b, bias,
                     out, M, N, K);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmv_rows_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                          const void* biases, const void* bias, void* out, int M, int N, int K,
                                          int group_size, int bits, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (!eagle_qmv_rows_supported(M, N, K)) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq)) return EAGLE_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const half_t* xh = static_cast<const half_t*>(x);
  const half_t* sh = static_cast<const half_t*>(scales);
  const half_t* bh = static_cast<const half_t*>(biases);
  const half_t* bi = static_cast<const half_t*>(bias);
  half_t* oh = static_cast<half_t*>(out);
  switch (qmv_rows_of(M)) {
    case 1: return qmv_launch<1>(xh, wq, sh, bh, bi, oh, M, N, K, st);
    case 2: return qmv_launch<2>(xh, wq, sh, bh, bi, oh, M, N, K, st);
    case 4: return qmv_launch<4>(xh, wq, sh, bh, bi, oh, M, N, K, st);
    default: return qmv_launch<8>(xh, wq, sh, bh, bi, oh, M, N, K, st);
  }
}

EAGLE_EXPORT int eagle_qmv_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                     const void* biases, const void* bias, void* out, int N, int K,
                                     int group_size, int bits, eagle_stream_t stream) {
  return eagle_qmv_rows_w4g64_f16(x, wq, scales, biases, bias, out, 1, N, K, group_size, bits, stream);
}
