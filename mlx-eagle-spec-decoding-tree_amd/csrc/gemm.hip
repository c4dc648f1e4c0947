// 4-bit group-64 quantised matmul for many rows (the prompt pass, mlx_eagle.py:522-533 through
// the QuantizedLinear layers of mlx_llama.py): out[M,N] = fp16( x[M,K] . (s*q + b)[N,K]^T ).
//
// With hundreds of rows the product is bound by the matrix cores, not by the weight stream, so
// this is a tiled GEMM: a workgroup of four waves owns a 128 x 128 output block, each wave a
// 64 x 64 quarter as 2 x 2 v_mfma_f32_32x32x16_f16 tiles (weights are the A operand: an
// accumulator lane then holds one output row and four consecutive columns per register
// group).  Per 64-wide K step (one quantisation group):
//   * the x block [128 x 64] goes through LDS (double buffered, one barrier per step), loaded
//     two steps ahead into registers;
//   * every lane loads the 16 bytes (four packed words = 32 weights) of its weight row that its
//     half of the MFMA K range needs, two steps ahead, and expands them in registers:
//     w & 0x000f000f | 0x64006400 is the fp16 pair (1024 + q0, 1024 + q4) (v_and_or_b32); minus
//     1024 (exact) and one packed fp16 fma with (s, b) gives the weights rounded to fp16, as
//     the reference kernels hold them.  That yields the eight weights of a word in the order
//     q0 q4 q1 q5 q2 q6 q3 q7; x is stored to LDS in the same order within every group of
//     eight, so both MFMA operands agree on which K index sits where.
// fp32 accumulation, one fp16 rounding, optional fp16 bias added after the rounding.
#include "common.h"

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int XS = BK + 8;                  // LDS row stride in halves (144 bytes: conflict-free 16-byte reads)

__device__ inline half8_t permute8(half8_t v) {
  return half8_t{v[0], v[4], v[1], v[5], v[2], v[6], v[3], v[7]};
}

__device__ inline uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(bits));
  return r;
}

// eight weights of one packed word, order q0 q4 q1 q5 q2 q6 q3 q7, as fp16(s*q + b).
// Even nibbles land in the low mantissa bits of 1024.0 (0x6400: one ulp = 1), odd nibbles four
// bits higher in 64.0 (0x5400: one ulp = 1/16), so only one shift is needed per word.
__device__ inline half8_t dequant_word(uint32_t w, half2_t s2, half2_t b2) {
  const half2_t k1024 = half2_t{(half_t)1024.f, (half_t)1024.f};
  const half2_t k64 = half2_t{(half_t)64.f, (half_t)64.f};
  union { uint32_t u; half2_t h; } c[4];
  const uint32_t w8 = w >> 8;
  c[0].u = and_or(w, 0x000f000fu, 0x64006400u);
  c[1].u = and_or(w, 0x00f000f0u, 0x54005400u);
  c[2].u = and_or(w8, 0x000f000fu, 0x64006400u);
  c[3].u = and_or(w8, 0x00f000f0u, 0x54005400u);
  half8_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t q = c[i].h - ((i & 1) ? k64 : k1024);      // exact
    const half2_t v = __builtin_elementwise_fma(q, s2, b2);
    o[2 * i] = v[0];
    o[2 * i + 1] = v[1];
  }
  return o;
}

__global__ __launch_bounds__(256) void qmm_gemm_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w, const half_t* __restrict__ s,
    const half_t* __restrict__ b, const half_t* __restrict__ bias, half_t* __restrict__ out, int M,
    int N, int K) {
  __shared__ __attribute__((aligned(16))) half_t xs[2][BM * XS];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int wn = wave & 1, wm = wave >> 1;
  const int n0 = blockIdx.x * BN + wn * 64;
  const int m0 = blockIdx.y * BM;
  const int KW = K >> 3;                    // packed words per weight row
  const int KG = K >> 6;                    // groups per weight row
  const int steps = K / BK;

  // x block loads: thread -> (row, 32-column half), four 16-byte pieces
  const int xr = tid >> 1, xh = tid & 1;
  int xrow = m0 + xr;
  if (xrow > M - 1) xrow = M - 1;           // rows past the end are never stored
  const half_t* xp = x + (long)xrow * K + xh * 32;
  // weight rows of this lane's two 32-row tiles
  int nrow[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    nrow[nt] = n0 + nt * 32 + ql;
    if (nrow[nt] > N - 1) nrow[nt] = N - 1;
  }

  // two register sets: the loads of step ks + 2 are issued while step ks is computed, so every
  // load has two steps to arrive even with a single wave per SIMD
  half8_t xreg[2][4];
  uint4_t wreg[2][2];
  half_t sreg[2][2], breg[2][2];
  auto fetch = [&](int ks, int p) {
#pragma unroll
    for (int g = 0; g < 4; ++g) xreg[p][g] = *reinterpret_cast<const half8_t*>(xp + (long)ks * BK + g * 8);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      wreg[p][nt] = *reinterpret_cast<const uint4_t*>(w + (long)nrow[nt] * KW + ks * 8 + hb * 4);
      sreg[p][nt] = s[(long)nrow[nt] * KG + ks];
      breg[p][nt] = b[(long)nrow[nt] * KG + ks];
    }
  };
  auto stash = [&](int buf, int p) {
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<half8_t*>(&xs[buf][xr * XS + xh * 32 + g * 8]) = permute8(xreg[p][g]);
  };

  float16_t acc[2][2];                      // [weight tile][x tile]
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;

  fetch(0, 0);
  fetch(steps > 1 ? 1 : 0, 1);
  stash(0, 0);
  __syncthreads();

  // One K step.  Register set p = ks & 1 holds the weights of step ks (its x part went to LDS
  // during the previous step); once they are expanded the set is free for step ks + 2.  The
  // loaded values are used where they were loaded: a copy of a register with a load in flight
  // would wait for the load.
  auto body = [&](int ks, int p) {
    half8_t af[2][4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const half2_t s2 = half2_t{sreg[p][nt], sreg[p][nt]}, b2 = half2_t{breg[p][nt], breg[p][nt]};
#pragma unroll
      for (int j = 0; j < 4; ++j) af[nt][j] = dequant_word(wreg[p][nt][j], s2, b2);
    }
    __builtin_amdgcn_sched_barrier(0);
    // unconditional (the last steps load their own data again): no branches in the loop body;
    // issued here, ahead of the matrix work (left alone, the scheduler sinks the loads to the
    // end of the step, where the in-order counter then waits for them at once)
    fetch(ks + 2 < steps ? ks + 2 : steps - 1, p);
    __builtin_amdgcn_sched_barrier(0);
    // all eight x operands of the step are requested at once: one LDS wait per step
    half8_t bf[4][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
        bf[j][mt] = *reinterpret_cast<const half8_t*>(&xs[p][(wm * 64 + mt * 32 + ql) * XS + hb * 32 + j * 8]);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[nt][j], bf[j][mt], acc[nt][mt], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    stash(p ^ 1, p ^ 1);
    __syncthreads();
  };
  int ks = 0;
  for (; ks + 1 < steps; ks += 2) {
    body(ks, 0);
    body(ks + 1, 1);
  }
  if (ks < steps) body(ks, 0);

  // accumulator register i of a lane: weight row (output column) 8*(i/4) + 4*hb + i%4 of the
  // tile, x row (output row) ql
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
    const int m = m0 + wm * 64 + mt * 32 + ql;
    if (m >= M) continue;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int n = n0 + nt * 32 + 8 * i4 + 4 * hb;
        if (n >= N) continue;                // N is a multiple of 4 columns (checked by the host)
        half4_t v = half4_t{(half_t)acc[nt][mt][4 * i4 + 0], (half_t)acc[nt][mt][4 * i4 + 1],
                            (half_t)acc[nt][mt][4 * i4 + 2], (half_t)acc[nt][mt][4 * i4 + 3]};
        if (bias) v += *reinterpret_cast<const half4_t*>(bias + n);
        *reinterpret_cast<half4_t*>(out + (long)m * N + n) = v;
      }
    }
  }
}

}  // namespace

EAGLE_EXPORT int eagle_qmm_gemm_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                          const void* biases, const void* bias, void* out, int M, int N,
                                          int K, int group_size, int bits, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (M < 1 || N < 8 || (N % 8) != 0 || K < 64 || (K % 64) != 0) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(out) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 7u)))
    return EAGLE_ERR_ALIGN;
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  hipLaunchKernelGGL(qmm_gemm_w4g64_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half_t*>(x), wq, static_cast<const half_t*>(scales),
                     static_cast<const half_t*>(biases), static_cast<const half_t*>(bias),
                     static_cast<half_t*>(out), M, N, K);
  return eagle_launch_status();
}
