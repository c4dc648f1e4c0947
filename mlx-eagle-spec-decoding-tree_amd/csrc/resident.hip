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
//
// A second kernel in this file chains two such products inside ONE launch of a resident grid
// (one workgroup per compute unit, all co-resident): the attention output projection with the
// residual add, then - across a grid-wide barrier - RMSNorm folded into the load of x, gate|up
// and SwiGLU (mlx_llama.py:195-196, 231-249, 214-215).  The weights of the second product are
// already on their way into the LDS ring while the first one runs and while the barrier is
// crossed, which is what a kernel boundary cannot do.

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
typedef __attribute__((address_space(3))) float lds_float;
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

// one quantised matrix [N, K] as the streaming waves see it
struct ResMat {
  const uint32_t* w;
  const half_t* s;
  const half_t* b;
  int N, K;
  int ntiles;          // 32-row weight tiles
  int pair;            // 1: workgroups take tiles in adjacent pairs
};

struct ResArgs {
  ResMat m;
  const half_t* x;
  const half_t* bias;
  half_t* out;
  int M;
};

// Tile i of workgroup wg: the workgroups take tiles (or adjacent pairs of tiles where there
// are many, so that a workgroup's consecutive output tiles fill whole 128-byte lines) round
// robin, so that at any moment the whole grid reads one contiguous stretch of the weight matrix
// (DRAM pages stay open; contiguous per-workgroup ranges measured 15 % slower).
__device__ inline int res_tile(int wg, int nwg, int i, int pair) {
  return ((wg + (i >> pair) * nwg) << pair) + (i & pair);
}
__device__ inline int res_count(int ntiles, int wg, int nwg, int pair) {
  int n = 0;
  for (int p = wg; (p << pair) < ntiles; p += nwg) n += pair && (p << 1) + 1 < ntiles ? 2 : 1;
  return n;
}

// Direct loads of one wave's unit of one tile into an 8 KB ring slot.  Load t: rows
// 8 (t / 2) + lane / 8, line t % 2 of the wave's 256-byte unit, 16-byte chunk
// (lane % 8) ^ ((row >> 1) & 7) of that line; it lands at slot + 1024 t + 16 lane.
__device__ inline void res_issue(const ResMat& m, int tile, lds_char* slot, int wave, int lane) {
  const int KW = m.K >> 3;
  const int lr = lane >> 3;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int r = 8 * (t >> 1) + lr;
    int row = tile * 32 + r;
    row = row < m.N ? row : m.N - 1;
    const int chunk = (lane & 7) ^ ((r >> 1) & 7);
    const uint32_t* src = m.w + (long)row * KW + wave * 64 + (t & 1) * 32 + chunk * 4;
    __builtin_amdgcn_global_load_lds(src, slot + t * 1024, 16, 0, 0);
  }
}

// The streaming waves' walk over `mine` tiles of matrix m.  Ring element e0 + i holds tile i
// (slot = element & 1) and has been requested before the call, as has element e0 + i + 1 where
// one exists; `issue_next(e)` requests ring element e (the caller knows which tile of which
// matrix that is and where the request has to stop).  On entry nothing but such requests may
// be outstanding in the wave.
template <class TileOf, class IssueNext>
__device__ inline void res_stream(const ResMat& m, int mine, int e0, TileOf tile_of, IssueNext issue_next,
                                  lds_char* ring, lds_float4* part, const half8_t (&xq)[8][4], int wave,
                                  int lane) {
  const int ql = lane & 31, hb = lane >> 5;
  const int G = m.K >> 6;
  // The lane's operand word of group g (row ql, chunk 2 g + hb of the unit): load
  // t = 2 (ql / 8) + g / 4, lane 8 (ql % 8) + (((2 g + hb) % 8) ^ ((ql >> 1) & 7)).
  int rd[8];
#pragma unroll
  for (int g = 0; g < 8; ++g)
    rd[g] = (2 * (ql >> 3) + (g >> 2)) * 1024 + 16 * (8 * (ql & 7) + (((2 * g + hb) & 7) ^ ((ql >> 1) & 7)));
  auto row_of = [&](int i) {
    const int r = tile_of(i < mine ? i : mine - 1) * 32 + ql;
    return r < m.N ? r : m.N - 1;
  };
  half8_t s8, b8, s8n, b8n;
  {
    const long r0 = row_of(0);
    s8 = *reinterpret_cast<const half8_t*>(m.s + r0 * G + wave * 8);
    b8 = *reinterpret_cast<const half8_t*>(m.b + r0 * G + wave * 8);
  }
  // scales of the first tile and every ring request made before the call
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  for (int i = 0; i < mine; ++i) {
    const int slot = (e0 + i) & 1;
    uint4_t wreg[8];
#pragma unroll
    for (int g = 0; g < 8; ++g)
      wreg[g] = *reinterpret_cast<lds_uint4*>(ring + slot * RES_TILE_BYTES + rd[g]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    {
      const long rn = row_of(i + 1);
      s8n = *reinterpret_cast<const half8_t*>(m.s + rn * G + wave * 8);
      b8n = *reinterpret_cast<const half8_t*>(m.b + rn * G + wave * 8);
    }
    issue_next(e0 + i + 2);
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
    // ring element e0 + i + 1 has landed: the scales of tile i + 1 and the eight loads of
    // element e0 + i + 2 came after it
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    s8 = s8n;
    b8 = b8n;
  }
}

// The reducing wave's side of res_stream: sum[i4][e] of tile i is the result for weight row
// 8 i4 + 4 hb + e of the tile and x row ql; `epilogue(i, sum)` stores it.
template <class Epilogue>
__device__ inline void res_reduce(int mine, int nws, lds_float4* part, int lane, Epilogue epilogue) {
  for (int i = 0; i < mine; ++i) {
    lds_only_barrier();
    lds_only_barrier();
    float4_t sum[4];
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) sum[i4] = float4_t{0.f, 0.f, 0.f, 0.f};
    const lds_float4* src = part + lane;
    for (int w = 0; w < nws; ++w)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) sum[i4] += src[(w * 4 + i4) * 64];
    epilogue(i, sum);
  }
}

// fp16 result (+ bias) of one tile, out [M, N]
__device__ inline void res_store_plain(const float4_t (&sum)[4], int tile, int lane, int M, int N,
                                       const half_t* bias, half_t* out) {
  const int ql = lane & 31, hb = lane >> 5;
  if (ql >= M) return;
#pragma unroll
  for (int i4 = 0; i4 < 4; ++i4) {
    const int n = tile * 32 + 8 * i4 + 4 * hb;
    if (n >= N) continue;
    half4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] = (half_t)sum[i4][e];
      if (bias) o[e] = o[e] + bias[n + e];
    }
    *reinterpret_cast<half4_t*>(out + (size_t)ql * N + n) = o;
  }
}

// SwiGLU of a (gate, up) tile pair: rows 0..15 of the tile are gate rows, 16..31 the matching
// up rows; out [M, N / 2]
__device__ inline void res_store_swiglu(const float4_t (&sum)[4], int tile, int lane, int M, int N,
                                        const half_t* bias, half_t* out) {
  const int ql = lane & 31, hb = lane >> 5;
  if (ql >= M) return;
  const int ldo = N >> 1;
#pragma unroll
  for (int i4 = 0; i4 < 2; ++i4) {
    const int c = 8 * i4 + 4 * hb;
    const int n_g = tile * 32 + c;
    if (n_g + 16 >= N) continue;
    half4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      half_t g = (half_t)sum[i4][e], u = (half_t)sum[i4 + 2][e];
      if (bias) {
        g = g + bias[n_g + e];
        u = u + bias[n_g + 16 + e];
      }
      const float gf = (float)g;
      const half_t act = (half_t)(gf / (1.0f + expf(-gf)));
      o[e] = (half_t)((float)act * (float)u);
    }
    *reinterpret_cast<half4_t*>(out + (size_t)ql * ldo + tile * 16 + c) = o;
  }
}

// a streaming wave's K unit of x: row ql, columns 512 wave + 64 g + 32 hb + 8 j .. + 8
__device__ inline void res_load_x(const half_t* x, int M, int K, int wave, int lane, half8_t (&xq)[8][4]) {
  const int ql = lane & 31, hb = lane >> 5;
  const int m = ql < M ? ql : M - 1;
  const half_t* xp = x + (long)m * K + wave * 512 + hb * 32;
#pragma unroll
  for (int g = 0; g < 8; ++g)
#pragma unroll
    for (int j = 0; j < 4; ++j) xq[g][j] = permute8(*reinterpret_cast<const half8_t*>(xp + g * 64 + j * 8));
}

template <bool SWIGLU>
__global__ __launch_bounds__(512) void qmm_res_w4g64_kernel(ResArgs a) {
  extern __shared__ __attribute__((aligned(16))) char res_lds[];
  lds_char* lds = (lds_char*)res_lds;
  const int wg = blockIdx.x, nwg = gridDim.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nws = a.m.K >> 9;
  const int mine = res_count(a.m.ntiles, wg, nwg, a.m.pair);
  if (mine == 0) return;
  lds_float4* part = reinterpret_cast<lds_float4*>(lds);
  auto tile_of = [&](int i) { return res_tile(wg, nwg, i, a.m.pair); };
  if (wave < nws) {
    lds_char* ring = lds + RES_PART_BYTES + wave * RES_RING_BYTES;
    auto issue = [&](int e) {
      res_issue(a.m, tile_of(e < mine ? e : mine - 1), ring + (e & 1) * RES_TILE_BYTES, wave, lane);
    };
    half8_t xq[8][4];
    res_load_x(a.x, a.M, a.m.K, wave, lane, xq);
    __builtin_amdgcn_sched_barrier(0);
    issue(0);
    issue(1);
    res_stream(a.m, mine, 0, tile_of, issue, ring, part, xq, wave, lane);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the clamped extra requests of the last tiles
  } else {
    res_reduce(mine, nws, part, lane, [&](int i, const float4_t (&sum)[4]) {
      if (SWIGLU)
        res_store_swiglu(sum, tile_of(i), lane, a.M, a.m.N, a.bias, a.out);
      else
        res_store_plain(sum, tile_of(i), lane, a.M, a.m.N, a.bias, a.out);
    });
  }
}

// ------------------------------------------------------------------------------------------
// Residual add + RMSNorm + gate|up + SwiGLU in one launch: the sum of the previous product's K
// slabs and the sums of squares first, spread over the whole grid, then - across a grid-wide
// barrier - the matmul with the norm folded into the load of x.
// ------------------------------------------------------------------------------------------
struct ChainArgs {
  ResMat gu;                // [2 I, D], gate and up rows interleaved in 16-row tiles
  const float* partial;     // [nslab][32][D] fp32 partial sums of the product that precedes the norm
  int nslab;
  half_t* h;                // [M, D] residual stream: read, updated in place (h += fp16(sum of slabs))
  const half_t* norm_w;     // [D]
  const half_t* gu_bias;    // [2 I] interleaved, or nullptr
  half_t* act;              // [M, I]
  float* ssq;               // [32 rows][segments] sums of squares, one 128-byte line each (scratch)
  unsigned* sync;           // [9 * 64] barrier counters (one line per group + one), never reset
  int* err;                 // set to 1 if the barrier gave up
  float eps;
  int M;
  long long spin_limit;     // 100 MHz ticks a workgroup waits at the barrier before giving up
};

// Grid-wide barrier of a resident grid, two levels (eight groups of workgroups, wg % 8), on
// counters that only ever grow: a workgroup learns which launch it belongs to from the value
// its own arrival returns, so nothing has to be reset between launches.  One wave of the
// workgroup (`signaller`: the one whose stores the others wait for; it has waited for them
// itself) arrives and polls; the other waves sleep at the workgroup barrier, which orders LDS
// only, so their outstanding weight requests stay in flight.  Waiting is bounded: after
// `limit` ticks the workgroup sets *err and returns false; the caller then skips the rest of
// its work and every wave still exits normally.
__device__ inline bool res_grid_barrier(unsigned* sync, int wg, int nwg, long long limit, int* err,
                                        bool signaller, lds_float* ok_flag) {
  if (signaller && (threadIdx.x & 63) == 0) {
    const unsigned ngrp = nwg < 8 ? nwg : 8;
    const unsigned grp = wg % ngrp;
    const unsigned members = nwg / ngrp + (grp < (unsigned)nwg % ngrp ? 1 : 0);
    unsigned* gcnt = sync + 64 + grp * 64;
    const unsigned old = __hip_atomic_fetch_add(gcnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned launch = old / members;                       // launches completed before this one
    if ((old + 1) % members == 0)
      __hip_atomic_fetch_add(sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned target = (launch + 1) * ngrp;
    const long long t0 = __builtin_amdgcn_s_memrealtime();
    float ok = 1.f;
    while ((int)(__hip_atomic_load(sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
      if (__builtin_amdgcn_s_memrealtime() - t0 > limit) {
        ok = 0.f;
        __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
    *ok_flag = ok;
  }
  lds_only_barrier();
  return *ok_flag != 0.f;
}

__global__ __launch_bounds__(512) void norm_mlp_in_kernel(ChainArgs a) {
  extern __shared__ __attribute__((aligned(16))) char res_lds[];
  lds_char* lds = (lds_char*)res_lds;
  const int wg = blockIdx.x, nwg = gridDim.x;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int D = a.gu.K;
  const int nws = D >> 9;
  lds_float4* part = reinterpret_cast<lds_float4*>(lds);
  const int n1 = res_count(a.gu.ntiles, wg, nwg, 0);
  auto gu_tile = [&](int i) { return res_tile(wg, nwg, i, 0); };
  lds_char* ring = lds + RES_PART_BYTES + (wave < nws ? wave : 0) * RES_RING_BYTES;
  auto issue = [&](int e) {
    res_issue(a.gu, gu_tile(e < n1 ? e : n1 - 1), ring + (e & 1) * RES_TILE_BYTES, wave, lane);
  };
  lds_char* nwl = lds + 1024 + (wave < nws ? wave : 0) * 1024;
  half8_t nw8 = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  if (wave < nws) nw8 = *reinterpret_cast<const half8_t*>(a.norm_w + wave * 512 + lane * 8);
  // the first two weight tiles are on their way before anything else happens
  if (wave < nws && n1 > 0) {
    issue(0);
    issue(1);
  }

  // ---- h += fp16(sum of the slabs), sums of squares: row wg / segs, segment wg % segs ----
  // (a segment is D / segs columns, a whole number of 128-byte lines: every line of h is
  // written by one compute unit only, so no L2 ever holds a line that is half stale)
  // (every streaming wave parks its 512 norm weights in LDS, in the idle time before the barrier)
  if (wave < nws) *reinterpret_cast<__attribute__((address_space(3))) half8_t*>(nwl + lane * 16) = nw8;
  // The wave that streams no weights does it (D / 8 / segs <= 64 lanes of eight columns), so that
  // the streaming waves' requests stay in flight across the barrier.
  const int segs = nwg / 32;                  // the grid is a multiple of 32 workgroups
  lds_float* flags = reinterpret_cast<lds_float*>(lds);      // [0..31] 1 / rms per row, [32] barrier result
  if (wave == nws) {
    const int row = wg / segs, seg = wg % segs;
    const int seg_cols = D / segs;
    float ss = 0.f;
    if (row < a.M && lane * 8 < seg_cols) {
      const size_t at = (size_t)row * D + seg * seg_cols + lane * 8;
      const half8_t v = eagle_slab_sum8(a.partial, a.nslab, (size_t)32 * D, at, nullptr);
      const half8_t r = *reinterpret_cast<const half8_t*>(a.h + at);
      half8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        o[e] = (half_t)((float)v[e] + (float)r[e]);
        ss += (float)o[e] * (float)o[e];
      }
      // written through to memory: the other compute units read it after the barrier
      const uint4_t bits = __builtin_bit_cast(uint4_t, o);
      unsigned long long* dst = reinterpret_cast<unsigned long long*>(a.h + at);
      __hip_atomic_store(dst, (unsigned long long)bits[0] | ((unsigned long long)bits[1] << 32), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + 1, (unsigned long long)bits[2] | ((unsigned long long)bits[3] << 32),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    ss = wave_sum(ss);
    if (lane == 0)
      __hip_atomic_store(a.ssq + (size_t)wg * 32, ss, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // the stores have been acknowledged
  }

  // ---- every workgroup has written its part of h ----
  if (!res_grid_barrier(a.sync, wg, nwg, a.spin_limit, a.err, wave == nws, flags + 32) || n1 == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  // ---- act = swiglu(norm(h) . Wgu^T) ----
  half8_t xq[8][4];
  lds_float* rstd = flags;
  if (wave == nws && lane < 32) {
    // 1 / rms of a row from the sums of its segments (one line each, owned by its writer)
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = k < segs ? a.ssq[(size_t)(lane * segs + k) * 32] : 0.f;
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) tot += v[k];
    rstd[lane] = 1.0f / sqrtf(tot / (float)D + a.eps);
  }
  if (wave < nws) {
    // the wave's K unit of h, all loads in flight together, in place in the operand registers
    const int m = ql < a.M ? ql : a.M - 1;
    const half_t* hp = a.h + (long)m * D + wave * 512 + hb * 32;
#pragma unroll
    for (int g = 0; g < 8; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) xq[g][j] = *reinterpret_cast<const half8_t*>(hp + g * 64 + j * 8);
  }
  lds_only_barrier();
  if (wave < nws) {
    const int m = ql < a.M ? ql : a.M - 1;
    const float rinv = rstd[m];
#pragma unroll
    for (int g = 0; g < 8; ++g) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half8_t w8 = *reinterpret_cast<__attribute__((address_space(3))) half8_t*>(
            nwl + (g * 64 + hb * 32 + j * 8) * 2);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)w8[e] * ((float)xq[g][j][e] * rinv));
        xq[g][j] = permute8(o);
      }
    }
  }
  lds_only_barrier();                                      // rstd has been read: the partial tiles may be written
  if (wave < nws) {
    res_stream(a.gu, n1, 0, gu_tile, issue, ring, part, xq, wave, lane);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    res_reduce(n1, nws, part, lane, [&](int i, const float4_t (&sum)[4]) {
      res_store_swiglu(sum, gu_tile(i), lane, a.M, a.gu.N, a.gu_bias, a.act);
    });
  }
}

int res_configure() {
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_res_w4g64_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, RES_LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_res_w4g64_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, RES_LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&norm_mlp_in_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, RES_LDS_BYTES) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  return EAGLE_OK;
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
  a.m.w = wq;
  a.m.s = static_cast<const half_t*>(scales);
  a.m.b = static_cast<const half_t*>(biases);
  a.m.N = N;
  a.m.K = K;
  a.m.ntiles = (N + 31) / 32;
  a.m.pair = a.m.ntiles >= 16 * RES_CU ? 1 : 0;
  a.x = static_cast<const half_t*>(x);
  a.bias = static_cast<const half_t*>(bias);
  a.out = static_cast<half_t*>(out);
  a.M = M;
  const int nws = K / 512;
  if (res_configure() != EAGLE_OK) return EAGLE_ERR_HIP;
  const int units = (a.m.ntiles + a.m.pair) >> a.m.pair;
  const int grid = units < RES_CU ? units : RES_CU;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (swiglu)
    hipLaunchKernelGGL(qmm_res_w4g64_kernel<true>, dim3(grid), dim3(64 * (nws + 1)), RES_LDS_BYTES, st, a);
  else
    hipLaunchKernelGGL(qmm_res_w4g64_kernel<false>, dim3(grid), dim3(64 * (nws + 1)), RES_LDS_BYTES, st, a);
  return eagle_launch_status();
}

EAGLE_EXPORT size_t eagle_norm_mlp_in_scratch_bytes(void) {
  // sums of squares: one 128-byte line per workgroup of the grid (256), then the barrier counters
  // (9 lines of 256 bytes)
  return (size_t)RES_CU * 128 + 9 * 256;
}

EAGLE_EXPORT int eagle_norm_mlp_in_supported(int M, int D, int I) {
  // 256 workgroups = 32 rows x 8 segments of D / 8 columns, each a whole number of 128-byte lines
  return M >= 1 && M <= EAGLE_MAX_M && D >= 512 && (D % 512) == 0 && D <= 512 * RES_MAX_WAVES && I >= 16 &&
         (I % 16) == 0;   // (D / 64 <= 64: one wave of eight-column lanes covers a segment)
}

EAGLE_EXPORT int eagle_norm_mlp_in_f16(const float* partial, int slabs, void* h, const void* norm_w, float eps,
                                       const uint32_t* gu_wq, const void* gu_scales, const void* gu_biases,
                                       const void* gu_bias, void* act, int M, int D, int I, void* scratch,
                                       size_t scratch_bytes, int* err_dev, long long spin_limit_ticks,
                                       eagle_stream_t stream) {
  if (!partial || !h || !norm_w || !gu_wq || !gu_scales || !gu_biases || !act || !scratch || !err_dev)
    return EAGLE_ERR_NULL;
  if (!eagle_norm_mlp_in_supported(M, D, I) || slabs < 1 || spin_limit_ticks < 1) return EAGLE_ERR_SHAPE;
  if (scratch_bytes < eagle_norm_mlp_in_scratch_bytes()) return EAGLE_ERR_WORKSPACE;
  const void* aligned[] = {partial, h, norm_w, gu_wq, gu_scales, gu_biases, act, scratch};
  for (const void* p : aligned)
    if (!eagle_aligned16(p)) return EAGLE_ERR_ALIGN;
  // one workgroup per compute unit: the grid has to be resident as a whole for the barrier
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return EAGLE_ERR_HIP;
  if (cus < RES_CU) return EAGLE_ERR_UNSUPPORTED;
  ChainArgs a;
  a.gu = ResMat{gu_wq, static_cast<const half_t*>(gu_scales), static_cast<const half_t*>(gu_biases), 2 * I, D,
                (2 * I) / 32, 0};
  a.partial = partial;
  a.nslab = slabs;
  a.h = static_cast<half_t*>(h);
  a.norm_w = static_cast<const half_t*>(norm_w);
  a.gu_bias = static_cast<const half_t*>(gu_bias);
  a.act = static_cast<half_t*>(act);
  a.ssq = static_cast<float*>(scratch);
  a.sync = reinterpret_cast<unsigned*>(static_cast<unsigned char*>(scratch) + (size_t)RES_CU * 128);
  a.err = err_dev;
  a.eps = eps;
  a.M = M;
  a.spin_limit = spin_limit_ticks;
  if (res_configure() != EAGLE_OK) return EAGLE_ERR_HIP;
  hipLaunchKernelGGL(norm_mlp_in_kernel, dim3(RES_CU), dim3(64 * (D / 512 + 1)), RES_LDS_BYTES,
                     static_cast<hipStream_t>(stream), a);
  return eagle_launch_status();
}
