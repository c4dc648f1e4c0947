// 4-bit group-64 quantised matmul for 1..32 rows of x with x RESIDENT IN REGISTERS and the K
// range split over the waves of a workgroup (same product and layout as csrc/qmm.hip;
// reference contract qmm_kernel.py:84-164, mlx_model_fwd_bench.py:65-73).
//
//   * One workgroup per compute unit.  Streaming wave w owns the K unit [512 w, 512 w + 512)
//     (eight quantisation groups) for the whole launch: it loads that unit of all 32 x rows
//     once, already in matrix-operand form (128 registers), and then walks over the
//     workgroup's 32-row weight tiles (round robin over the grid, in adjacent pairs where
//     there are many).
//   * Weights travel HBM -> LDS by direct loads (global_load_lds_dwordx4: no registers, no
//     wait in the issuing wave).  One instruction moves eight rows x one 128-byte line, so a
//     wave's request touches eight cache lines instead of the 32 that a load in
//     matrix-operand layout (one row per lane) touches: the rate of line requests, not bytes,
//     is what bounded that form (3.9 TB/s with the arithmetic removed).  The 16-byte chunks of
//     a line are XOR-swizzled with the row index on the way in, so that the later ds_read_b128
//     in operand layout (lane = row, half-group) is free of bank conflicts.  Each wave keeps
//     two tiles (16 KB) in flight or waiting in its private LDS ring: the tile after next is
//     requested as soon as the current one has been copied to registers.
//   * Expansion: a shift and a mask leave each nibble pair in mantissa bits 6..9 of two fp16
//     SUBNORMALS (q * 2^-18, exact); one packed fma with (s * 2^18, b) gives fp16(s q + b)
//     with a single rounding and no offset to subtract: three instructions per weight pair.
//     s * 2^18 must stay below 65504 (s < 0.2499); beyond that the output is inf / NaN.
//     The words of a register expand in the order q0 q4 q1 q5 q2 q6 q3 q7, and x is held in
//     the same order.  v_mfma_f32_32x32x16_f16 with the weights as the A operand: four per
//     group and wave.
//   * Every streaming wave leaves its 32 x 32 fp32 partial tile in LDS (two LDS-only barriers
//     per tile: one before the partials are overwritten, one after they are written).  One
//     further wave adds the partials in wave order, rounds to fp16, adds the bias (or applies
//     SwiGLU to a (gate, up) tile pair that the interleaved layout puts into the same lanes)
//     and stores, while the streaming waves work on the next tile.
//   * Whole K per workgroup: no K slabs, no workspace, no counters.  K is a multiple of 512 and
//     at most 3584 (seven streaming waves + the reducing wave = 512 threads, two waves per SIMD,
//     256 registers each).  LDS: 28 KB of partial tiles + 16 KB of weight ring per wave.
#include "common.h"

namespace {

constexpr int RES_MAX_WAVES = 7;            // streaming waves (K units of 512)
constexpr int RES_CU = 256;
constexpr int RES_PART_BYTES = RES_MAX_WAVES * 4 * 64 * 16;      // one partial tile per streaming wave
constexpr int RES_RING_TILES = 2;
constexpr int RES_TILE_BYTES = 8 * 1024;                         // one wave's unit of one tile
constexpr int RES_RING_BYTES = RES_RING_TILES * RES_TILE_BYTES;  // per streaming wave
constexpr int RES_LDS_BYTES = RES_PART_BYTES + RES_MAX_WAVES * RES_RING_BYTES;

typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) float4_t lds_float4;
typedef __attribute__((address_space(3))) uint4_t lds_uint4;

__device__ inline void lds_only_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ inline half8_t permute8(half8_t v) {
  return half8_t{v[0], v[4], v[1], v[5], v[2], v[6], v[3], v[7]};
}

// eight weights of a packed word as fp16(s q + b), order q0 q4 q1 q5 q2 q6 q3 q7;
// s18 = (s * 2^18, s * 2^18)
__device__ inline half8_t dequant_word_sub(uint32_t w, half2_t s18, half2_t b2) {
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

struct ResArgs {
  const half_t* x;
  const uint32_t* w;
  const half_t* s;
  const half_t* b;
  const half_t* bias;
  half_t* out;
  int M, N, K;
  int ntiles;          // 32-row weight tiles
  int pair;            // 1: workgroups take tiles in adjacent pairs
};

// Tile i of workgroup wg: the workgroups take tiles in adjacent pairs, round robin, so that at
// any moment the whole grid reads one contiguous stretch of the weight matrix (DRAM pages stay
// open; contiguous per-workgroup ranges measured 15 % slower) and a workgroup's consecutive
// output tiles fill whole 128-byte lines.
// (`pair` = 0: single tiles, for matrices with fewer than two tiles per workgroup.)
__device__ inline int res_tile(int wg, int nwg, int i, int pair) {
  return ((wg + (i >> pair) * nwg) << pair) + (i & pair);
}
__device__ inline int res_count(int ntiles, int wg, int nwg, int pair) {
  int n = 0;
  for (int p = wg; (p << pair) < ntiles; p += nwg) n += pair && (p << 1) + 1 < ntiles ? 2 : 1;
  return n;
}

// lds: RES_LDS_BYTES
template <bool SWIGLU>
__device__ inline void res_matmul(const ResArgs& a, int wg, int nwg, lds_char* lds) {
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int nws = a.K >> 9;
  const int G = a.K >> 6, KW = a.K >> 3;
  const int mine = res_count(a.ntiles, wg, nwg, a.pair);
  if (mine == 0) return;
  lds_float4* part = reinterpret_cast<lds_float4*>(lds);

  if (wave < nws) {
    lds_char* ring = lds + RES_PART_BYTES + wave * RES_RING_BYTES;
    // Direct load t of a tile: rows 8 (t / 2) + lane / 8, line t % 2 of the wave's 256-byte
    // unit, 16-byte chunk (lane % 8) ^ ((row >> 1) & 7) of that line; it lands at
    // slot + 1024 t + 16 lane.
    const int lr = lane >> 3;
    auto issue = [&](int i, int slot) {
      const int tile = res_tile(wg, nwg, i < mine ? i : mine - 1, a.pair);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int r = 8 * (t >> 1) + lr;
        int row = tile * 32 + r;
        row = row < a.N ? row : a.N - 1;
        const int chunk = (lane & 7) ^ ((r >> 1) & 7);
        const uint32_t* src = a.w + (long)row * KW + wave * 64 + (t & 1) * 32 + chunk * 4;
        __builtin_amdgcn_global_load_lds(src, ring + slot * RES_TILE_BYTES + t * 1024, 16, 0, 0);
      }
    };
    // The lane's operand word of group g (row ql, chunk 2 g + hb of the unit): load
    // t = 2 (ql / 8) + g / 4, lane 8 (ql % 8) + (((2 g + hb) % 8) ^ ((ql >> 1) & 7)).
    int rd[8];
#pragma unroll
    for (int g = 0; g < 8; ++g)
      rd[g] = (2 * (ql >> 3) + (g >> 2)) * 1024 + 16 * (8 * (ql & 7) + (((2 * g + hb) & 7) ^ ((ql >> 1) & 7)));
    auto row_of = [&](int i) {
      const int r = res_tile(wg, nwg, i < mine ? i : mine - 1, a.pair) * 32 + ql;
      return r < a.N ? r : a.N - 1;
    };
    // this wave's K unit of x: row ql, columns 512 wave + 64 g + 32 hb + 8 j .. + 8
    half8_t xq[8][4];
    {
      const int m = ql < a.M ? ql : a.M - 1;
      const half_t* xp = a.x + (long)m * a.K + wave * 512 + hb * 32;
#pragma unroll
      for (int g = 0; g < 8; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) xq[g][j] = permute8(*reinterpret_cast<const half8_t*>(xp + g * 64 + j * 8));
    }
    half8_t s8, b8, s8n, b8n;
    {
      const long r0 = row_of(0);
      s8 = *reinterpret_cast<const half8_t*>(a.s + r0 * G + wave * 8);
      b8 = *reinterpret_cast<const half8_t*>(a.b + r0 * G + wave * 8);
    }
    __builtin_amdgcn_sched_barrier(0);
    issue(0, 0);
    issue(1, 1);
    // everything issued so far has landed except (at most) the second tile's eight loads
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    for (int i = 0; i < mine; ++i) {
      const int slot = i & 1;
      uint4_t wreg[8];
#pragma unroll
      for (int g = 0; g < 8; ++g)
        wreg[g] = *reinterpret_cast<lds_uint4*>(ring + slot * RES_TILE_BYTES + rd[g]);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      {
        const long rn = row_of(i + 1);
        s8n = *reinterpret_cast<const half8_t*>(a.s + rn * G + wave * 8);
        b8n = *reinterpret_cast<const half8_t*>(a.b + rn * G + wave * 8);
      }
      issue(i + 2, slot);
      __builtin_amdgcn_sched_barrier(0);
      float16_t acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        const half_t sc = (half_t)((float)s8[g] * 262144.f);
        const half_t bi = b8[g];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const half8_t af = dequant_word_sub(wreg[g][j], half2_t{sc, sc}, half2_t{bi, bi});
          acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, xq[g][j], acc, 0, 0, 0);
        }
      }
      lds_only_barrier();                    // the reducing wave has read the previous partials
      lds_float4* dst = part + (wave * 4) * 64 + lane;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        dst[i4 * 64] = float4_t{acc[4 * i4], acc[4 * i4 + 1], acc[4 * i4 + 2], acc[4 * i4 + 3]};
      lds_only_barrier();                    // partials of tile i are in LDS
      // tile i + 1 has landed: the scales of tile i + 1 and the loads of tile i + 2 came after it
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      s8 = s8n;
      b8 = b8n;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the clamped extra loads of the last tiles
  } else {
    // the reducing wave
    const int ldo = SWIGLU ? a.N >> 1 : a.N;
    for (int i = 0; i < mine; ++i) {
      lds_only_barrier();
      lds_only_barrier();
      const int tile = res_tile(wg, nwg, i, a.pair);
      float4_t sum[4];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) sum[i4] = float4_t{0.f, 0.f, 0.f, 0.f};
      const lds_float4* src = part + lane;
      for (int w = 0; w < nws; ++w)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) sum[i4] += src[(w * 4 + i4) * 64];
      // register 4 i4 + e of the lane: weight row 8 i4 + 4 hb + e of the tile, x row ql
      if (ql >= a.M) continue;
      if (SWIGLU) {
        // rows 0..15 of the tile are gate rows, 16..31 the matching up rows
#pragma unroll
        for (int i4 = 0; i4 < 2; ++i4) {
          const int c = 8 * i4 + 4 * hb;
          const int n_g = tile * 32 + c;
          if (n_g + 16 >= a.N) continue;
          half4_t o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            half_t g = (half_t)sum[i4][e], u = (half_t)sum[i4 + 2][e];
            if (a.bias) {
              g = g + a.bias[n_g + e];
              u = u + a.bias[n_g + 16 + e];
            }
            const float gf = (float)g;
            const half_t act = (half_t)(gf / (1.0f + expf(-gf)));
            o[e] = (half_t)((float)act * (float)u);
          }
          *reinterpret_cast<half4_t*>(a.out + (size_t)ql * ldo + tile * 16 + c) = o;
        }
      } else {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          const int n = tile * 32 + 8 * i4 + 4 * hb;
          if (n >= a.N) continue;
          half4_t o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            o[e] = (half_t)sum[i4][e];
            if (a.bias) o[e] = o[e] + a.bias[n + e];
          }
          *reinterpret_cast<half4_t*>(a.out + (size_t)ql * ldo + n) = o;
        }
      }
    }
  }
}

template <bool SWIGLU>
__global__ __launch_bounds__(512) void qmm_res_w4g64_kernel(ResArgs a) {
  extern __shared__ __attribute__((aligned(16))) char res_lds[];
  res_matmul<SWIGLU>(a, blockIdx.x, gridDim.x, (lds_char*)res_lds);
}

}  // namespace

EAGLE_EXPORT int eagle_qmm_res_supported(int M, int N, int K) {
  return M >= 1 && M <= EAGLE_MAX_M && N >= 8 && (N % 8) == 0 && K >= 512 && (K % 512) == 0 &&
         K <= 512 * RES_MAX_WAVES;
}

EAGLE_EXPORT int eagle_qmm_res_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                         const void* biases, const void* bias, void* out, int M, int N,
                                         int K, int group_size, int bits, int swiglu, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (!eagle_qmm_res_supported(M, N, K)) return EAGLE_ERR_SHAPE;
  if (swiglu && (N % 32) != 0) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(scales) || !eagle_aligned16(biases) ||
      (reinterpret_cast<uintptr_t>(out) & 7u) || (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  ResArgs a;
  a.x = static_cast<const half_t*>(x);
  a.w = wq;
  a.s = static_cast<const half_t*>(scales);
  a.b = static_cast<const half_t*>(biases);
  a.bias = static_cast<const half_t*>(bias);
  a.out = static_cast<half_t*>(out);
  a.M = M;
  a.N = N;
  a.K = K;
  a.ntiles = (N + 31) / 32;
  const int nws = K / 512;
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_res_w4g64_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, RES_LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_res_w4g64_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, RES_LDS_BYTES) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  a.pair = a.ntiles >= 4 * RES_CU ? 1 : 0;
  const int units = (a.ntiles + a.pair) >> a.pair;
  const int grid = units < RES_CU ? units : RES_CU;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (swiglu)
    hipLaunchKernelGGL(qmm_res_w4g64_kernel<true>, dim3(grid), dim3(64 * (nws + 1)), RES_LDS_BYTES, st, a);
  else
    hipLaunchKernelGGL(qmm_res_w4g64_kernel<false>, dim3(grid), dim3(64 * (nws + 1)), RES_LDS_BYTES, st, a);
  return eagle_launch_status();
}
