// 4-bit (group 64) quantised matmul for M = 1..32 rows of x, gfx950.
//
//   out[m,n] = fp16( sum_k x[m,k] * (s[n,k/64] * q[n,k] + b[n,k/64]) )
//
// Weight layout is the MLX one: wq[N, K/8] uint32, nibble i of a word is element
// 8*word + i; scales/biases [N, K/64] fp16.  (Reference contract:
// qmm_kernel.py:84-164, kernels/progression/simd_no_swizzle_cast.metal.)
//
// Structure: a weight streamer with x resident in registers.
//
//  * A workgroup owns one K slab and a contiguous range of 16-row weight tiles.  Each of
//    its `nw` streaming waves owns one column unit of the slab (256 columns for M <= 16,
//    128 for M <= 32) for the whole launch: it loads that unit of x ONCE, straight into
//    MFMA operand registers, and then walks down the rows.  Per tile a lane issues one or
//    two 128-bit loads; the four lanes that share a row read 64 contiguous bytes per
//    instruction and the waves of the workgroup together read whole rows.  Four tiles are
//    in flight per wave in a register ring.
//  * Nibbles are expanded with the fp16 magic-number trick only:
//    (w & 0x000f000f) | 0x6400 = 1024 + q and (w & 0x00f000f0) | 0x5400 = 64 + q give the
//    pairs (q0,q4) (q1,q5) (q2,q6) (q3,q7) as MFMA operands without subtracting the offsets
//    or applying scale and bias per weight.  v_mfma_f32_16x16x32_f16 accumulates one
//    quantisation group at a time, t[m,n] = sum_k x[m,k] (off_k + q[n,k]); the group result
//    is folded in with one fp32 FMA per accumulator, acc += s[n,g] * t.  What that leaves,
//        sum_g b[n,g] * xs[m,g]  -  sum_g s[n,g] * (1024 * xsE[m,g] + 64 * xsO[m,g])
//    (xs = per-group sums of x, over even / odd columns), is one more MFMA per tile whose
//    x-side operand is computed once per launch (split into fp16 high and low parts, so
//    that it carries 22 bits) and whose weight-side operand is the tile's scales and biases.
//    v_permlane32_swap regroups the loaded words so that all four lanes of a row feed one
//    quantisation group per MFMA.
//  * Scales and biases of a batch of tiles are staged through LDS by the streaming waves
//    (whole row segments, coalesced) one batch ahead.
//  * Each streaming wave leaves its 16 x M partial tile in LDS; two further waves of the
//    workgroup only add the partials in wave order and store the results, one batch
//    behind the streamers (double-buffered, one barrier per batch).  Streaming waves
//    therefore never have stores in flight and their prefetch ring is waited on exactly.
//  * K slabs (blockIdx.y), needed when K exceeds what 14 waves cover, are added through
//    fp32 partials in a workspace: the last workgroup of a tile range to arrive sums the
//    slabs in slab order, so results are deterministic.  The partials travel as
//    device-scope relaxed atomics (write-through stores, L2-bypassing loads): no L2
//    write-back / invalidate fence, which costs microseconds on a multi-XCD part.
#include "common.h"

#include <mutex>

namespace {

constexpr int MAX_STREAM_WAVES = 14;   // + 2 reducing waves = 1024 threads
constexpr int NWR = 2;                 // reducing waves per workgroup
constexpr int MAX_WIDE_WAVES = 10;     // 32 rows x 256 columns of x need 168 registers: 12 waves per CU
constexpr int MAX_SPLITS = 64;
constexpr int MAX_RANGES = EAGLE_QMM_COUNTER_BYTES / 4;
constexpr int LDS_MAX = 160 * 1024;
constexpr int NUM_CU = 256;

__device__ inline half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ inline uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// (v & mask) | bits in one VALU op.  The compiler splits the two-literal form into
// v_and + v_or; holding `bits` in a VGPR and `mask` in an SGPR makes it encodable.
__device__ inline uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(bits));
  return r;
}

// 8 nibbles of one packed word -> fp16 (1024+q0, 1024+q4, 64+q1, 64+q5, 1024+q2, 1024+q6,
// 64+q3, 64+q7): five VALU operations.
__device__ inline half8_t expand8(uint32_t v, uint32_t magic_lo, uint32_t magic_hi) {
  const uint32_t v2 = v >> 8;
  uint4_t u;
  u[0] = and_or(v, 0x000f000fu, magic_lo);
  u[1] = and_or(v, 0x00f000f0u, magic_hi);
  u[2] = and_or(v2, 0x000f000fu, magic_lo);
  u[3] = and_or(v2, 0x00f000f0u, magic_hi);
  return __builtin_bit_cast(half8_t, u);
}

// Exchange the upper 32 lanes of `a` with the lower 32 lanes of `b`.
__device__ inline void swap32(uint32_t& a, uint32_t& b) {
  const uint2_t r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load (vmcnt(0)), which would drain the prefetch ring at each batch.
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int NT, int GW>
struct Cfg {
  static constexpr int RING = 4;                // tiles in flight per streaming wave
  static constexpr int B = 4 / NT;              // tiles per batch (one barrier per batch)
  static constexpr int BPS = RING / B;          // batches per super-step of RING tiles
  static constexpr int CW = GW * 64;            // columns owned by a streaming wave
  static constexpr int NL = GW / 2;             // 128-bit weight loads per lane per tile
  static constexpr int NMF = GW * 2;            // MFMAs per 16 rows of x per tile
  static constexpr int UNIT = GW * 2;           // bytes of scales (or biases) per row per wave
  static constexpr int SB_ARRAY = 16 * B * 16 * UNIT;   // LDS bytes: one array, one buffer
  static constexpr int SB_BUF = 2 * SB_ARRAY;
  static constexpr int NSU = B / 2;             // staging units per streaming thread per batch
};

__host__ __device__ inline int pbuf_bytes(int nw) { return 2 * nw * 4096; }

struct Launch {
  int nw;       // streaming waves per workgroup
  int phases;   // column units a streaming wave owns, one after the other
  int splits;   // K slabs (gridDim.y); a slab is nw * phases units
  int ranges;   // tile ranges (gridDim.x)
  int wide = 0; // M > 16 only: 256-column units, at most MAX_WIDE_WAVES streaming waves
};

template <int V>
struct Mode { static constexpr int value = V; };
constexpr int STEP_MID = 0;    // more tiles of this phase follow: reload the ring from it
constexpr int STEP_NEXT = 1;   // last super-step of a phase, another phase follows
constexpr int STEP_LAST = 2;   // last super-step of the last phase: nothing to prefetch

// NT: 16-row blocks of x (1 or 2).  GW: quantisation groups per streaming wave and phase.
// SLOWSB: scales / biases are fetched element by element (odd group counts, rows shorter
// than a unit, unaligned arrays).
template <int NT, int GW, bool SLOWSB>
__global__ __launch_bounds__(NT == 2 && GW == 4 ? 768 : 1024) void qmm_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w,
    const half_t* __restrict__ s, const half_t* __restrict__ b,
    const half_t* __restrict__ bias, half_t* __restrict__ out,
    float* __restrict__ partial, unsigned* __restrict__ counters,
    int M, int N, int K, int nw, int phases, int t_q, int t_r, int swiglu) {
  using C = Cfg<NT, GW>;
  constexpr int B = C::B;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  float4_t* pbuf4 = reinterpret_cast<float4_t*>(lds);                 // [2][nw][256] float4
  unsigned char* sbuf = lds + pbuf_bytes(nw);                         // [2][2][16B][16] units
  float4_t* accl4 = reinterpret_cast<float4_t*>(sbuf + 2 * C::SB_BUF); // [batches][256] float4

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane & 15;   // x row (A operand) / weight row of the tile (B operand)
  const int h = lane >> 4;   // K block of the MFMA this lane feeds
  const int G = K >> 6;
  const int K8 = K >> 3;
  const int nsplit = gridDim.y;
  const int slab = blockIdx.y;
  const int tiles_total = (N + 15) >> 4;
  const int bx = blockIdx.x;
  // ranges are counted in tiles, or in (gate, up) tile pairs for the SwiGLU form
  const int gran = swiglu ? 2 : 1;
  const int t_lo = gran * (bx * t_q + (bx < t_r ? bx : t_r));
  const int t_hi = t_lo + gran * (t_q + (bx < t_r ? 1 : 0));
  const int nss = (t_hi - t_lo + C::RING - 1) / C::RING;   // super-steps per phase
  const int nbp = nss * C::BPS;                             // batches per phase
  const bool to_out = nsplit == 1;

  if (wave < nw) {
    // ------------------------------------------------------------------ streaming wave
    const uint32_t magic_lo = 0x64006400u, magic_hi = 0x54005400u;
    const uint32_t row_bytes = (uint32_t)K8 * 4u;
    const int unit0 = slab * phases * nw + wave;            // this wave's unit in phase 0

    // Weight addresses are (uniform tile base) + (32-bit lane offset), which the loads take as
    // scalar base + vector offset: no per-tile address arithmetic in the vector unit.  The lane
    // offset is row-in-tile * row bytes + the byte offset of this lane's words inside the row
    // (clamped into the row); it changes only with the column unit.  Rows past N in a last,
    // partial tile read the last row instead.
    const int rows_last = N - 16 * (tiles_total - 1);                 // 8 or 16
    const uint32_t r_last = (uint32_t)(r < rows_last ? r : rows_last - 1);
    auto unit_woff = [&](int unit, uint32_t (&o)[2 * C::NL]) {
#pragma unroll
      for (int ld = 0; ld < C::NL; ++ld) {
        int word = unit * (C::CW / 8) + ld * 16 + h * 4;
        if (word > K8 - 4) word = K8 - 4;
        o[ld] = (uint32_t)r * row_bytes + (uint32_t)word * 4u;
        o[C::NL + ld] = r_last * row_bytes + (uint32_t)word * 4u;
      }
    };
    const unsigned char* wbytes = reinterpret_cast<const unsigned char*>(w);
    const size_t tile_bytes = (size_t)16 * row_bytes;
    auto load_w = [&](int tile, const uint32_t (&o)[2 * C::NL], uint4_t (&dst)[C::NL]) {
      const int t = tile < t_hi ? tile : t_hi - 1;
      const unsigned char* tb = wbytes + (size_t)t * tile_bytes;      // uniform
      const bool last = t == tiles_total - 1;                         // uniform
#pragma unroll
      for (int ld = 0; ld < C::NL; ++ld)
        dst[ld] = *reinterpret_cast<const uint4_t*>(tb + (last ? o[C::NL + ld] : o[ld]));
    };

    // ---- scale / bias staging: this thread's units of a batch (16*B rows x nw units x 2 arrays)
    const int nthr_s = nw * 64;
    int su_row[C::NSU], su_c[C::NSU], su_lds[C::NSU];
    const half_t* su_arr[C::NSU];
    const float inv_nw = 1.0f / (float)nw;
#pragma unroll
    for (int k = 0; k < C::NSU; ++k) {
      // NT == 1: two units per thread, unit k of array k.  NT == 2: one unit, array = upper half.
      const int a = NT == 1 ? k : (tid >= 32 * nw ? 1 : 0);
      const int rem = NT == 1 ? tid : tid - a * 32 * nw;
      int row = (int)(((float)rem + 0.5f) * inv_nw);
      if (row * nw > rem) --row;
      if ((row + 1) * nw <= rem) ++row;
      const int c = rem - row * nw;
      su_row[k] = row;
      su_c[k] = c;
      su_arr[k] = a ? b : s;
      su_lds[k] = ((a * 16 * B + row) * 16 + (c ^ (row & 15))) * C::UNIT;
    }
    // Staged values travel in registers from the load to the LDS store.  The vmcnt counter
    // retires loads in order, so waiting for a staged value also waits for every weight load
    // issued before it: the staging load must be at least as old as the ring slot consumed
    // at the time of the store.  With two batches per super-step (NT == 2) that takes a
    // lookahead of two batches and two register sets.
    constexpr int NSET = NT == 2 ? C::BPS : 1;
    uint2_t su_vals[NSET][C::NSU];
    auto stage_load = [&](int tile0, int ph, uint2_t (&su_val)[C::NSU]) {
#pragma unroll
      for (int k = 0; k < C::NSU; ++k) {
        int row = tile0 * 16 + su_row[k];
        if (row > N - 1) row = N - 1;
        const half_t* p = su_arr[k] + (size_t)row * G;
        int g0 = ((slab * phases + ph) * nw + su_c[k]) * GW;
        if (SLOWSB) {
          half_t v[4];
#pragma unroll
          for (int e = 0; e < GW; ++e) {
            int g = g0 + e;
            if (g > G - 1) g = G - 1;
            v[e] = p[g];
          }
          half2_t lo = {v[0], v[1]};
          su_val[k][0] = as_u32(lo);
          if (GW == 4) {
            half2_t hi = {v[2], v[3]};
            su_val[k][1] = as_u32(hi);
          }
        } else {
          if (g0 > G - GW) g0 = G - GW;
          if (GW == 4) su_val[k] = *reinterpret_cast<const uint2_t*>(p + g0);
          else su_val[k][0] = *reinterpret_cast<const uint32_t*>(p + g0);
        }
      }
    };
    auto stage_store = [&](int buf, const uint2_t (&su_val)[C::NSU]) {
#pragma unroll
      for (int k = 0; k < C::NSU; ++k) {
        unsigned char* q = sbuf + buf * C::SB_BUF + su_lds[k];
        if (GW == 4) *reinterpret_cast<uint2_t*>(q) = su_val[k];
        else *reinterpret_cast<uint32_t*>(q) = su_val[k][0];
      }
    };

    // ---- x side: this wave's unit of x as MFMA operands, and the operand of the bias /
    // offset MFMA: K block 0 carries the group sums of x (high and low fp16 parts), K block 1
    // carries -(16 * even sum + odd sum); the other two blocks are zero.
    half8_t xop[NT][C::NMF];
    half8_t xaux[NT];
    const int hperm = ((h & 1) << 2) | (h & 2);          // 0, 4, 2, 6
    uint4_t xraw[NT][C::NMF];
    auto x_issue = [&](int unit) {
      const int col0 = unit * C::CW;
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < C::NMF; ++j) {
          const int wi = 16 * (j >> 2) + 8 * ((j >> 1) & 1) + (j & 1) + hperm;
          // out-of-range rows and columns read a valid address and are zeroed afterwards
          int col = col0 + 8 * wi;
          if (col > K - 8) col = K - 8;
          int m = 16 * t + r;
          if (m > M - 1) m = M - 1;
          xraw[t][j] = *reinterpret_cast<const uint4_t*>(x + (size_t)m * K + col);
        }
    };
    auto x_finish = [&](int unit) {
      const int col0 = unit * C::CW;
      float sE[NT][GW], sO[NT][GW];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g = 0; g < GW; ++g) sE[t][g] = sO[t][g] = 0.f;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int j = 0; j < C::NMF; ++j) {
          const int wi = 16 * (j >> 2) + 8 * ((j >> 1) & 1) + (j & 1) + hperm;
          const int col = col0 + 8 * wi;
          const int m = 16 * t + r;
          uint4_t u = xraw[t][j];
          if (!(m < M && col < K)) u = uint4_t{0u, 0u, 0u, 0u};
          uint4_t o;
          o[0] = __builtin_amdgcn_perm(u[2], u[0], 0x05040100u);   // (x0, x4)
          o[1] = __builtin_amdgcn_perm(u[2], u[0], 0x07060302u);   // (x1, x5)
          o[2] = __builtin_amdgcn_perm(u[3], u[1], 0x05040100u);   // (x2, x6)
          o[3] = __builtin_amdgcn_perm(u[3], u[1], 0x07060302u);   // (x3, x7)
          xop[t][j] = __builtin_bit_cast(half8_t, o);
          const half2_t e0 = as_h2(o[0]), o0 = as_h2(o[1]), e1 = as_h2(o[2]), o1 = as_h2(o[3]);
          sE[t][j >> 1] += ((float)e0[0] + (float)e0[1]) + ((float)e1[0] + (float)e1[1]);
          sO[t][j >> 1] += ((float)o0[0] + (float)o0[1]) + ((float)o1[0] + (float)o1[1]);
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        half8_t a;
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = (half_t)0.f;
#pragma unroll
        for (int g = 0; g < GW; ++g) {
          float se = sE[t][g], so = sO[t][g];
          se += __shfl_xor(se, 16, 64);
          se += __shfl_xor(se, 32, 64);
          so += __shfl_xor(so, 16, 64);
          so += __shfl_xor(so, 32, 64);
          const float v = h == 0 ? se + so : -(16.f * se + so);
          const half_t hi = (half_t)v;
          const half_t lo = (half_t)(v - (float)hi);
          a[g] = h < 2 ? hi : (half_t)0.f;
          a[4 + g] = h < 2 ? lo : (half_t)0.f;
        }
        xaux[t] = a;
      }
    };
    auto load_x = [&](int unit) {
      x_issue(unit);
      x_finish(unit);
    };
    const half2_t kmul = h == 0 ? half2_t{(half_t)1.f, (half_t)1.f} : half2_t{(half_t)64.f, (half_t)64.f};

    // ---- prologue.  Loads retire in issue order, so the small ones go first: x (cached, it
    // was just written) and the first scales / biases arrive while the weight ring, which
    // takes microseconds to fill, is in flight, and the x operands are built in that shadow.
    stage_load(t_lo, 0, su_vals[0]);
    if (NT == 2) {
#pragma unroll
      for (int q = 1; q < NSET; ++q) stage_load(t_lo + q * B < t_hi ? t_lo + q * B : t_lo, 0, su_vals[q]);
    }
    x_issue(unit0);
    uint32_t woff[2 * C::NL];
    unit_woff(unit0, woff);
    uint4_t ring[C::RING][C::NL];
    __builtin_amdgcn_sched_barrier(0);      // keep the issue order: the scheduler would sink the ring
#pragma unroll
    for (int p = 0; p < C::RING; ++p) load_w(t_lo + p, woff, ring[p]);
    __builtin_amdgcn_sched_barrier(0);
    x_finish(unit0);
    stage_store(0, su_vals[0]);
    lds_barrier();

    // One tile: bias / offset MFMA, then per quantisation group two MFMAs and the scale FMAs.
    auto tile_compute = [&](const uint4_t (&wq)[C::NL], int sbuf_idx, int pbuf_idx, int j) {
      const unsigned char* sp = sbuf + sbuf_idx * C::SB_BUF + (((j * 16 + r) * 16) + (wave ^ r)) * C::UNIT;
      uint2_t sv, bv;
      if (GW == 4) {
        sv = *reinterpret_cast<const uint2_t*>(sp);
        bv = *reinterpret_cast<const uint2_t*>(sp + C::SB_ARRAY);
      } else {
        sv[0] = *reinterpret_cast<const uint32_t*>(sp);
        bv[0] = *reinterpret_cast<const uint32_t*>(sp + C::SB_ARRAY);
        sv[1] = sv[0];
        bv[1] = bv[0];
      }
      // weight-side operand of the bias / offset MFMA: biases in K block 0, 64 * scales in
      // K block 1 (blocks 2 and 3 meet zeros)
      uint4_t aux;
      {
        const half2_t s0 = as_h2(sv[0]) * kmul, s1 = as_h2(sv[1]) * kmul;
        const uint32_t q0 = h == 0 ? bv[0] : as_u32(s0);
        const uint32_t q1 = h == 0 ? bv[1] : as_u32(s1);
        aux[0] = q0; aux[1] = q1; aux[2] = q0; aux[3] = q1;
      }
      float4_t acc[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            xaux[t], __builtin_bit_cast(half8_t, aux), float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
      for (int ld = 0; ld < C::NL; ++ld) {
        uint32_t q[4] = {wq[ld][0], wq[ld][1], wq[ld][2], wq[ld][3]};
        swap32(q[0], q[2]);
        swap32(q[1], q[3]);
#pragma unroll
        for (int gl = 0; gl < 2; ++gl) {
          const int g = 2 * ld + gl;
          float4_t tt[NT];
#pragma unroll
          for (int t = 0; t < NT; ++t) tt[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int pp = 0; pp < 2; ++pp) {
            const half8_t wop = expand8(q[2 * gl + pp], magic_lo, magic_hi);
#pragma unroll
            for (int t = 0; t < NT; ++t)
              tt[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xop[t][4 * ld + 2 * gl + pp], wop,
                                                             tt[t], 0, 0, 0);
          }
          const half_t sg = as_h2(sv[g >> 1])[g & 1];
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][i] = __builtin_fmaf((float)sg, tt[t][i], acc[t][i]);
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t)
        pbuf4[(pbuf_idx * nw + wave) * 256 + (j * NT + t) * 64 + lane] = acc[t];
    };

    // ---- main loop over super-steps of RING tiles (ring slots are compile-time indices) and
    // phases.  Every load of the loop is unconditional: targets beyond the work are
    // redirected to addresses that are already cached.
    // (the host guarantees at least one tile per workgroup and one phase: a loop that always
    // runs once keeps the ring loads of the prologue where they are, before the x operands)
    const int nvs = phases * nss;
    int ph = 0, ss = 0, vs = 0;
    do {
      const bool last_ss = ss == nss - 1;
      const bool more_phases = ph + 1 < phases;
      if (ss == 0 && ph > 0) load_x(unit0 + ph * nw);
      if (last_ss && more_phases) unit_woff(unit0 + (ph + 1) * nw, woff);   // reloads now target the next phase
      const int tb = t_lo + C::RING * ss;
      const int nbase = last_ss ? (more_phases ? t_lo : t_hi) : tb + C::RING;
#pragma unroll
      for (int p = 0; p < C::RING; ++p) {
        const int j = p % B;                       // tile inside its batch
        const int bq = p / B;
        const int buf = (vs * C::BPS + bq) & 1;    // batch parity over all phases
        if (j == 0) {
          // scales and biases of a later batch: the next one (NT == 1) or the same batch of
          // the next super-step (NT == 2)
          int n_tile0 = NT == 1 ? tb + p + B : tb + C::RING + p, n_ph = ph;
          if ((NT == 2 || bq == C::BPS - 1) && last_ss) {
            n_tile0 = NT == 1 ? t_lo : t_lo + p;
            n_ph = ph + 1;
          }
          if (n_ph >= phases || n_tile0 >= t_hi) {   // no such batch: fetch the current one again
            n_tile0 = tb + p;
            n_ph = ph;
          }
          stage_load(n_tile0, n_ph, su_vals[NT == 2 ? bq : 0]);
        }
        if (tb + p < t_hi) tile_compute(ring[p], buf, buf, j);
        load_w(nbase + p, woff, ring[p]);
        if (j == B - 1) {
          stage_store(buf ^ 1, su_vals[NT == 2 ? (bq + 1) % C::BPS : 0]);
          lds_barrier();
        }
      }
      if (++ss == nss) {
        ss = 0;
        ++ph;
      }
    } while (++vs < nvs);
  } else {
    // ------------------------------------------------------------------ reducing wave
    // A batch is four 16 x 16 blocks (tile j of the batch, x block t), block jt = j * NT + t;
    // MFMA lane ln of a block holds out[16 t + 4 (ln / 16) + i][tile * 16 + ln % 16], i = 0..3.
    // Reducing wave ww owns MFMA lanes 32 ww .. 32 ww + 31 of every block, i.e. rows
    // 16 t + 8 ww .. + 7 of all tiles of the batch: after a transpose through 1 KiB of LDS
    // each of its lanes stores eight consecutive columns of one row (16 bytes), and the lanes
    // of a row cover all tiles of the batch.  A lane sums two blocks per batch: with one x
    // block (NT == 1) tiles it and it + 2 for the lane halves, with two (NT == 2) tile it of
    // x block = lane half.  Either way a lane's two blocks are neighbouring tiles, which is
    // what the SwiGLU form needs: gate in slot 0, up in slot 1.
    // The whole workgroup waits at the next barrier for these two waves: they go first
    // whenever they have something to issue.
    __builtin_amdgcn_s_setprio(3);
    const int ww = wave - nw;                 // 0 .. 1
    const int hi = lane >> 5;
    const int ln = (lane & 31) + 32 * ww;     // MFMA lane
    const int rr0 = 4 * ((ln >> 4) & 1);      // first of this lane's four rows inside the wave's eight
    const int cc = ln & 15;
    int sl_l4[2], sl_j[2];
    float* sl_part[2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int j = NT == 1 ? (swiglu ? 2 * hi + it : it + 2 * hi) : it;
      const int t = NT == 1 ? 0 : hi;
      sl_j[it] = j;
      sl_l4[it] = (j * NT + t) * 64 + ln;
      // partial[slab][tile][t][i][64]
      sl_part[it] = partial + (((size_t)slab * tiles_total * NT + t) * 4) * 64 + ln;
    }
    // Output staging of this wave: rows (t, rr) x the columns of the batch, fp16, 1 KiB.  It
    // reuses the slots this wave has just summed: the halves (MFMA lanes 32 ww ..) of blocks
    // 0 and 1 of the first streaming wave's partial, 512 bytes each, which nobody else reads
    // and the streaming waves do not write again before the next barrier.
    const int ocols = swiglu ? 8 * B : 16 * B;               // output columns per batch
    constexpr int RPR = 4 * NT;                              // staged rows per 512-byte region
    auto ost = [&](const float4_t* pb, int row, int col) -> half_t* {
      unsigned char* base = reinterpret_cast<unsigned char*>(const_cast<float4_t*>(pb)) +
                            ((row / RPR) * 64 + 32 * ww) * 16;
      return reinterpret_cast<half_t*>(base) + (row % RPR) * ocols + col;
    };
    const int st_t = NT == 1 ? 0 : hi;
    // where this lane's 16-byte piece of the staged rows goes
    const int lpr = ocols / 8;                               // lanes per row
    const int o_row = lane / lpr;                            // 0 .. 8 NT - 1 (when active)
    const int o_col = (lane % lpr) * 8;
    const bool o_active = lane < 8 * NT * lpr;
    const int o_m = 16 * (o_row >> 3) + 8 * ww + (o_row & 7);
    const int ldo = swiglu ? N >> 1 : N;
    lds_barrier();
    for (int ph = 0; ph < phases; ++ph) {
      for (int bi = 0; bi < nbp; ++bi) {
        lds_barrier();
        const int buf = (ph * nbp + bi) & 1;
        const int tile0 = t_lo + bi * B;
        const float4_t* pb = pbuf4 + buf * nw * 256;
        float4_t sums[2];
        bool live[2];
#pragma unroll
        for (int it = 0; it < 2; ++it) {
          const int tile = tile0 + sl_j[it];
          live[it] = tile < t_hi;
          if (!live[it]) continue;
          const float4_t* src = pb + sl_l4[it];
          float4_t sum;
          if (nw == MAX_STREAM_WAVES) {
            // the common shape: all partials fetched with immediate offsets before the adds
            float4_t v[MAX_STREAM_WAVES];
#pragma unroll
            for (int wv = 0; wv < MAX_STREAM_WAVES; ++wv) v[wv] = src[wv * 256];
            sum = v[0];
#pragma unroll
            for (int wv = 1; wv < MAX_STREAM_WAVES; ++wv) sum += v[wv];
          } else {
            sum = src[0];
            for (int wv = 1; wv < nw; ++wv) sum += src[wv * 256];
          }
          if (phases > 1) {
            float4_t* a = accl4 + bi * 256 + sl_l4[it];
            if (ph > 0) sum += *a;
            if (ph + 1 < phases) {
              *a = sum;
              live[it] = false;
            }
          }
          sums[it] = sum;
        }
        if (!to_out) {
#pragma unroll
          for (int it = 0; it < 2; ++it) {
            if (!live[it]) continue;
            float* dst = sl_part[it] + (size_t)(tile0 + sl_j[it]) * (NT * 256);
#pragma unroll
            for (int i = 0; i < 4; ++i)
              __hip_atomic_store(dst + i * 64, sums[it][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          continue;
        }
        if (ph + 1 < phases) continue;
        // fp16 results into the staging rows
        if (swiglu) {
          // slots 0 and 1 of this lane are the gate tile and the up tile of one pair
          if (live[0] && live[1]) {
            const int n_g = (tile0 + sl_j[0]) * 16 + cc;
            half_t bg = (half_t)0.f, bu = (half_t)0.f;
            if (bias && n_g + 16 < N) {
              bg = bias[n_g];
              bu = bias[n_g + 16];
            }
            const int pcol = (sl_j[0] >> 1) * 16 + cc;       // pair inside the batch
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              half_t g = (half_t)sums[0][i], u = (half_t)sums[1][i];
              if (bias) {
                g = g + bg;
                u = u + bu;
              }
              const float gf = (float)g;
              const half_t a = (half_t)(gf / (1.0f + expf(-gf)));
              *ost(pb, st_t * 8 + rr0 + i, pcol) = (half_t)((float)a * (float)u);
            }
          }
        } else {
#pragma unroll
          for (int it = 0; it < 2; ++it) {
            if (!live[it]) continue;
            const int n = (tile0 + sl_j[it]) * 16 + cc;
            half_t bn = (half_t)0.f;
            if (bias && n < N) bn = bias[n];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              half_t r = (half_t)sums[it][i];
              if (bias) r = r + bn;
              *ost(pb, st_t * 8 + rr0 + i, sl_j[it] * 16 + cc) = r;
            }
          }
        }
        // the staged rows are private to this wave: its own LDS writes are enough to wait for
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (o_active && o_m < M) {
          // column of the piece in the output: tiles (or pairs) of the batch side by side
          const int unit0 = swiglu ? tile0 >> 1 : tile0;
          const int n0 = unit0 * 16 + o_col;
          const int t_of = swiglu ? tile0 + 2 * (o_col >> 4) + 1 : tile0 + (o_col >> 4);
          if (t_of < t_hi && n0 < ldo) {
            const half8_t v = *reinterpret_cast<const half8_t*>(ost(pb, o_row, o_col));
            *reinterpret_cast<half8_t*>(out + (size_t)o_m * ldo + n0) = v;
          }
        }
      }
    }
  }

  if (nsplit > 1) {
    // ---- the last workgroup of this tile range to arrive adds the slabs, in slab order
    int* flag = reinterpret_cast<int*>(lds);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's partial stores are done
    __syncthreads();
    if (tid == 0) {
      const unsigned old = __hip_atomic_fetch_add(&counters[blockIdx.x], 1u, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT);
      *flag = old == (unsigned)(nsplit - 1);
      if (old == (unsigned)(nsplit - 1))
        __hip_atomic_store(&counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (*flag) {
      // one thread per (tile, x block, row, half of the 16 columns): its eight values are
      // consecutive floats of every slab's partial and become one 16-byte store.  In the
      // SwiGLU form an item is a (gate, up) tile pair and the store is the activation.
      const int per_tile = NT * 256;                       // floats
      const int items = ((t_hi - t_lo) / gran) * NT * 32;
      const size_t slab_stride = (size_t)tiles_total * per_tile;
      auto sum_slabs = [&](const float* src, float (&v)[8]) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
        for (int sp0 = 0; sp0 < nsplit; sp0 += 4) {        // sixteen loads in flight, added in slab order
          uint64_t pv[4][4];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const int sp = sp0 + k < nsplit ? sp0 + k : nsplit - 1;
            const uint64_t* q = reinterpret_cast<const uint64_t*>(src + sp * slab_stride);
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2)
              pv[k][e2] = __hip_atomic_load(q + e2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (sp0 + k < nsplit) {
#pragma unroll
              for (int e2 = 0; e2 < 4; ++e2) {
                union { uint64_t u; float f[2]; } cv;
                cv.u = pv[k][e2];
                v[2 * e2] += cv.f[0];
                v[2 * e2 + 1] += cv.f[1];
              }
            }
        }
      };
      for (int idx = tid; idx < items; idx += blockDim.x) {
        const int tile = t_lo + gran * (idx / (NT * 32));
        const int rem = idx % (NT * 32);
        const int t = rem >> 5;
        const int row = (rem >> 1) & 15;                   // row of the x block
        const int hc = rem & 1;
        const int m = 16 * t + row;
        const int n0 = tile * 16 + 8 * hc;
        // floats (t*4 + i)*64 + 16*rg + c with row = 4 rg + i, c = 8 hc .. 8 hc + 7
        const float* src = partial + (size_t)tile * per_tile + (t * 4 + (row & 3)) * 64 + 16 * (row >> 2) + 8 * hc;
        float v[8];
        sum_slabs(src, v);
        if (swiglu) {
          float u[8];
          sum_slabs(src + per_tile, u);                    // the up tile follows the gate tile
          if (n0 + 16 < N + 8 && m < M) {
            half8_t o;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              half_t g = (half_t)v[e], uu = (half_t)u[e];
              if (bias) {
                g = g + bias[n0 + e];
                uu = uu + bias[n0 + 16 + e];
              }
              const float gf = (float)g;
              const half_t a = (half_t)(gf / (1.0f + expf(-gf)));
              o[e] = (half_t)((float)a * (float)uu);
            }
            *reinterpret_cast<half8_t*>(out + (size_t)m * (N >> 1) + (tile >> 1) * 16 + 8 * hc) = o;
          }
        } else if (n0 < N && m < M) {
          half8_t o;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            o[e] = (half_t)v[e];
            if (bias) o[e] = o[e] + bias[n0 + e];
          }
          *reinterpret_cast<half8_t*>(out + (size_t)m * N + n0) = o;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
inline int nt_of(int M) { return M <= 16 ? 1 : 2; }
inline int cw_of(int M, int wide = 0) { return (M <= 16 || wide) ? 256 : 128; }
constexpr int MAX_PHASES = 8;

// gran = 1: ranges are counted in tiles; gran = 2: in (gate, up) tile pairs
int lds_bytes(int M, int N, const Launch& L, int gran = 1) {
  const int sb = M <= 16 ? 2 * Cfg<1, 4>::SB_BUF
                         : (L.wide ? 2 * Cfg<2, 4>::SB_BUF : 2 * Cfg<2, 2>::SB_BUF);
  int acc = 0;
  if (L.phases > 1) {
    const int tiles = (N + 15) / 16 / gran;
    const int per_range = gran * ((tiles + L.ranges - 1) / L.ranges);
    acc = (per_range + 3) / 4 * 4 * nt_of(M) * 1024;        // fp32 16 x M per tile, whole super-steps
  }
  return pbuf_bytes(L.nw) + sb + acc;
}

int validate_launch(int M, int N, int K, const Launch& L, int gran = 1) {
  if (L.nw < 1 || L.nw > MAX_STREAM_WAVES || L.splits < 1 || L.splits > MAX_SPLITS ||
      L.phases < 1 || L.phases > MAX_PHASES)
    return EAGLE_ERR_SHAPE;
  if (L.wide && (M <= 16 || L.nw > MAX_WIDE_WAVES)) return EAGLE_ERR_SHAPE;
  const int units = (K + cw_of(M, L.wide) - 1) / cw_of(M, L.wide);
  const long per_slab = (long)L.nw * L.phases;
  if (per_slab * L.splits < units || per_slab * (L.splits - 1) >= units) return EAGLE_ERR_SHAPE;
  const int tiles = (N + 15) / 16 / gran;
  if (L.ranges < 1 || L.ranges > tiles || L.ranges > MAX_RANGES) return EAGLE_ERR_SHAPE;
  if (lds_bytes(M, N, L, gran) > LDS_MAX) return EAGLE_ERR_SHAPE;
  return EAGLE_OK;
}

size_t partial_bytes(int M, int N, int splits) {
  if (splits <= 1) return 0;
  const size_t tiles = (N + 15) / 16;
  return (size_t)splits * tiles * nt_of(M) * 256 * sizeof(float);
}

// Launch shape.  A workgroup covers nw * phases column units; K slabs beyond that cost a
// round trip of fp32 partials, so there are only as many as 14 waves x 2 phases force, or as
// it takes to give every compute unit a workgroup when there are few row tiles.  Tile ranges:
// about one workgroup per compute unit, more when the per-range accumulators of a
// multi-phase launch would not fit LDS.
// The busiest workgroup sets the time: no more ranges than it takes to keep its share
// (items = tiles, or tile pairs in the SwiGLU form).
inline int balanced_ranges(int items, int ranges) {
  const int most = (items + ranges - 1) / ranges;
  return (items + most - 1) / most;
}

void choose(int M, int N, int K, Launch* out) {
  const int tiles = (N + 15) / 16;
  Launch L;
  if (M > 16) {
    // 256-column units on fewer, fatter waves (A/B runs of a whole verify step): when K needs
    // slabs anyway (K > 3584) they remove the second phase; with very many tiles they halve
    // the per-tile overhead of the two phases.  Smaller shapes are faster on 14 narrow waves.
    const int uw = (K + 255) / 256;
    const int un = (K + 127) / 128;
    if (tiles >= 16 * NUM_CU && uw > MAX_WIDE_WAVES / 2 && uw <= 2 * MAX_WIDE_WAVES) {
      L.wide = 1;                        // very many tiles: partials would be a large matrix
      L.phases = 2;
      L.nw = (uw + 1) / 2;
      L.splits = 1;
    } else if (un > 2 * MAX_STREAM_WAVES && !(tiles < 3 * NUM_CU / 2 && un <= 4 * MAX_STREAM_WAVES)) {
      // (few tiles and K up to 7168: four narrow slabs, below)
      L.wide = 1;
      L.phases = 1;
      const int least = (uw + MAX_WIDE_WAVES - 1) / MAX_WIDE_WAVES;
      // of the slab counts close to the least possible, the one that gives the most workgroups
      // (tile ranges x slabs) up to one per compute unit
      int best = least, best_wgs = 0;
      for (int sp = least; sp <= least + 2 && sp <= uw; ++sp) {
        int r = NUM_CU / sp;
        if (r < 1) r = 1;
        if (r > tiles) r = tiles;
        const int wgs = sp * balanced_ranges(tiles, r);
        if (wgs > best_wgs) {
          best_wgs = wgs;
          best = sp;
        }
      }
      L.splits = best;
      L.nw = (uw + L.splits - 1) / L.splits;
      L.splits = (uw + L.nw - 1) / L.nw;
    }
    if (L.wide) {
      int ranges = NUM_CU / L.splits;
      if (ranges < 1) ranges = 1;
      if (ranges > tiles) ranges = tiles;
      if (ranges > MAX_RANGES) ranges = MAX_RANGES;
      L.ranges = ranges;
      while (lds_bytes(M, N, L) > LDS_MAX && L.ranges < tiles && L.ranges < MAX_RANGES) ++L.ranges;
      L.ranges = balanced_ranges(tiles, L.ranges);
      *out = L;
      return;
    }
  }
  const int units = (K + cw_of(M) - 1) / cw_of(M);
  // M <= 16: one phase only (a phase switch costs more than a K slab there)
  const int phase_cap = M <= 16 ? 1 : 2;
  int splits = (units + phase_cap * MAX_STREAM_WAVES - 1) / (phase_cap * MAX_STREAM_WAVES);
  int fill = tiles >= 160 ? 1 : (NUM_CU + tiles - 1) / tiles;
  if (fill > 4) fill = 4;
  // About one tile per compute unit: four slabs of a few waves, each walking several tiles,
  // beat fewer slabs of many waves that touch one or two tiles
  if (tiles < 3 * NUM_CU / 2 && units >= (M <= 16 ? 8 : 16)) fill = 4;
  // K of at most 1024: a slab would be one or two waves; the round trip of the partials costs
  // more than the idle compute units (4.8 us against 6.7 us for 1152 x 896 at 8 rows)
  if (units <= (M <= 16 ? 4 : 8)) fill = 1;
  if (splits < fill) splits = fill;
  // With only a few tiles per workgroup a second phase is mostly start-up latency (new x, a
  // drained ring); two K slabs on twice the workgroups finish sooner.  (With more tiles the
  // two forms time alike in isolation and the phases win inside a verify step.)
  if (splits == 1 && units > MAX_STREAM_WAVES && tiles < 4 * NUM_CU) splits = 2;
  if (splits > units) splits = units;
  int per_slab = (units + splits - 1) / splits;
  L.phases = (per_slab + MAX_STREAM_WAVES - 1) / MAX_STREAM_WAVES;
  L.nw = (per_slab + L.phases - 1) / L.phases;
  // 64-byte units (M > 16): two neighbouring waves share each 128-byte line of a weight row,
  // so an even wave count keeps every line inside one phase (left alone when the slabs divide
  // the units exactly)
  if (M > 16 && (L.nw & 1) && L.nw < MAX_STREAM_WAVES && (units % splits) != 0) ++L.nw;
  per_slab = L.nw * L.phases;
  L.splits = (units + per_slab - 1) / per_slab;
  int ranges = NUM_CU / L.splits;
  if (ranges < 1) ranges = 1;
  if (ranges > tiles) ranges = tiles;
  if (ranges > MAX_RANGES) ranges = MAX_RANGES;
  L.ranges = ranges;
  while (lds_bytes(M, N, L) > LDS_MAX && L.ranges < tiles && L.ranges < MAX_RANGES) {
    L.ranges += NUM_CU / L.splits > 0 ? NUM_CU / L.splits : 1;
    if (L.ranges > tiles) L.ranges = tiles;
  }
  L.ranges = balanced_ranges(tiles, L.ranges);
  *out = L;
}

template <int NT, int GW, bool SLOWSB>
int launch(const void* x, const uint32_t* wq, const void* s, const void* b, const void* bias,
           void* out, float* partial, unsigned* counters, int M, int N, int K, const Launch& L,
           int swiglu, hipStream_t stream) {
  const int lds = lds_bytes(M, N, L, swiglu ? 2 : 1);
  static bool attr_set = false;   // more than 64 KB of LDS needs an explicit opt-in, once
  if (lds > 65536 && !attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_w4g64_kernel<NT, GW, SLOWSB>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_MAX) != hipSuccess)
      return EAGLE_ERR_HIP;
    attr_set = true;
  }
  const int tiles = ((N + 15) / 16) / (swiglu ? 2 : 1);      // range units: tiles or tile pairs
  hipLaunchKernelGGL((qmm_w4g64_kernel<NT, GW, SLOWSB>), dim3(L.ranges, L.splits),
                     dim3(64 * (L.nw + NWR)), lds, stream, (const half_t*)x, wq,
                     (const half_t*)s, (const half_t*)b, (const half_t*)bias, (half_t*)out,
                     partial, counters, M, N, K, L.nw, L.phases, tiles / L.ranges, tiles % L.ranges, swiglu);
  return eagle_launch_status();
}

int validate(const void* x, const uint32_t* wq, const void* s, const void* b, const void* bias,
             void* out, int M, int N, int K) {
  if (!x || !wq || !s || !b || !out) return EAGLE_ERR_NULL;
  if (M < 1 || M > EAGLE_MAX_M || N < 8 || (N % 8) != 0 || K < 64 || (K % 64) != 0)
    return EAGLE_ERR_SHAPE;
  if ((long)K > (long)cw_of(M) * MAX_STREAM_WAVES * 2 * MAX_SPLITS) return EAGLE_ERR_SHAPE;
  if ((long)N * (K / 2) >= (1L << 32)) return EAGLE_ERR_SHAPE;   // 32-bit byte offsets
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(out) ||
      (reinterpret_cast<uintptr_t>(s) & 1u) || (reinterpret_cast<uintptr_t>(b) & 1u) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  return EAGLE_OK;
}

int run(const void* x, const uint32_t* wq, const void* scales, const void* biases,
        const void* bias, void* out, int M, int N, int K, const Launch& L, int swiglu,
        void* workspace, size_t workspace_bytes, hipStream_t st) {
  float* partial = nullptr;
  unsigned* counters = nullptr;
  if (L.splits > 1) {
    if (!workspace || !eagle_aligned16(workspace) ||
        workspace_bytes < (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, N, L.splits))
      return EAGLE_ERR_WORKSPACE;
    counters = reinterpret_cast<unsigned*>(workspace);
    partial = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) +
                                       EAGLE_QMM_COUNTER_BYTES);
  }
  // vector fetches of scales / biases need whole, aligned units in every row
  const int G = K / 64;
  const int gw = (M <= 16 || L.wide) ? 4 : 2;
  const uintptr_t amask = gw == 4 ? 7u : 3u;
  const bool slow = (G % gw) != 0 || (reinterpret_cast<uintptr_t>(scales) & amask) ||
                    (reinterpret_cast<uintptr_t>(biases) & amask);
  if (M <= 16)
    return slow ? launch<1, 4, true>(x, wq, scales, biases, bias, out, partial, counters, M, N, K, L, swiglu, st)
                : launch<1, 4, false>(x, wq, scales, biases, bias, out, partial, counters, M, N, K, L, swiglu, st);
  if (L.wide)
    return slow ? launch<2, 4, true>(x, wq, scales, biases, bias, out, partial, counters, M, N, K, L, swiglu, st)
                : launch<2, 4, false>(x, wq, scales, biases, bias, out, partial, counters, M, N, K, L, swiglu, st);
  return slow ? launch<2, 2, true>(x, wq, scales, biases, bias, out, partial, counters, M, N, K, L, swiglu, st)
              : launch<2, 2, false>(x, wq, scales, biases, bias, out, partial, counters, M, N, K, L, swiglu, st);
}

}  // namespace

EAGLE_EXPORT size_t eagle_qmm_workspace_bytes(int M, int N, int K) {
  if (M < 1 || M > EAGLE_MAX_M || N < 1 || K < 64) return 0;
  Launch L;
  choose(M, N, K, &L);
  return (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, N, L.splits);
}

EAGLE_EXPORT size_t eagle_qmm_workspace_bytes_tuned(int M, int N, int splits) {
  if (M < 1 || M > EAGLE_MAX_M || N < 1 || splits < 1) return 0;
  return (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, N, splits);
}

EAGLE_EXPORT int eagle_qmm_plan(int M, int N, int K, int* plan5) {
  if (!plan5) return EAGLE_ERR_NULL;
  if (M < 1 || M > EAGLE_MAX_M || N < 8 || K < 64 || (K % 64) != 0) return EAGLE_ERR_SHAPE;
  Launch L;
  choose(M, N, K, &L);
  plan5[0] = L.nw; plan5[1] = L.phases; plan5[2] = L.splits; plan5[3] = L.ranges;
  plan5[4] = cw_of(M, L.wide);
  return EAGLE_OK;
}

EAGLE_EXPORT int eagle_qmm_w4g64_f16_tuned(const void* x, const uint32_t* wq, const void* scales,
                                           const void* biases, const void* bias, void* out, int M,
                                           int N, int K, int nw, int phases, int splits, int ranges,
                                           int unit_cols, void* workspace, size_t workspace_bytes,
                                           eagle_stream_t stream) {
  int rc = validate(x, wq, scales, biases, bias, out, M, N, K);
  if (rc != EAGLE_OK) return rc;
  if (unit_cols != 0 && unit_cols != 128 && unit_cols != 256) return EAGLE_ERR_SHAPE;
  if (unit_cols == 128 && M <= 16) return EAGLE_ERR_SHAPE;
  Launch L{nw, phases, splits, ranges};
  L.wide = (unit_cols == 256 && M > 16) ? 1 : 0;
  rc = validate_launch(M, N, K, L);
  if (rc != EAGLE_OK) return rc;
  return run(x, wq, scales, biases, bias, out, M, N, K, L, 0, workspace, workspace_bytes,
             static_cast<hipStream_t>(stream));
}

EAGLE_EXPORT int eagle_qmm_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                     const void* biases, const void* bias, void* out, int M,
                                     int N, int K, int group_size, int bits, void* workspace,
                                     size_t workspace_bytes, eagle_stream_t stream) {
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  int rc = validate(x, wq, scales, biases, bias, out, M, N, K);
  if (rc != EAGLE_OK) return rc;
  Launch L;
  choose(M, N, K, &L);
  rc = validate_launch(M, N, K, L);
  if (rc != EAGLE_OK) return rc;
  return run(x, wq, scales, biases, bias, out, M, N, K, L, 0, workspace, workspace_bytes,
             static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------------------------------------
// The same matmul for callers that cannot allocate: the split-K workspace is a fixed array in
// device memory that belongs to the library.
// ------------------------------------------------------------------------------------------
namespace {

constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)EAGLE_QMM_NOALLOC_SCRATCH_BYTES;
constexpr int NOALLOC_MAX_DEVICES = 64;

// Every GPU the library runs on holds its own copy of this array, at its own address, until
// the process ends.  In host code the name is only a handle for hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

__global__ void zero_u32_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// device address of `scratch` on the current device, looked up once per device
int noalloc_scratch(void** out) {
  static void* ptrs[NOALLOC_MAX_DEVICES];
  static bool known[NOALLOC_MAX_DEVICES];
  static std::mutex lock;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return EAGLE_ERR_HIP;
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return EAGLE_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> guard(lock);
  if (!known[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return EAGLE_ERR_HIP;
    ptrs[dev] = p;
    known[dev] = true;
  }
  *out = ptrs[dev];
  return EAGLE_OK;
}

}  // namespace

EAGLE_EXPORT size_t eagle_qmm_noalloc_scratch_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

EAGLE_EXPORT int eagle_qmm_w4g64_f16_noalloc(const void* x, const uint32_t* wq, const void* scales,
                                             const void* biases, const void* bias, void* out, int M,
                                             int N, int K, int group_size, int bits,
                                             eagle_stream_t stream) {
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  int rc = validate(x, wq, scales, biases, bias, out, M, N, K);
  if (rc != EAGLE_OK) return rc;
  Launch L;
  choose(M, N, K, &L);
  rc = validate_launch(M, N, K, L);
  if (rc != EAGLE_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  void* ws = nullptr;
  size_t ws_bytes = 0;
  if (L.splits > 1) {
    ws_bytes = (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, N, L.splits);
    if (ws_bytes > NOALLOC_SCRATCH_BYTES) return EAGLE_ERR_WORKSPACE;   // shape needs more than the fixed array
    rc = noalloc_scratch(&ws);
    if (rc != EAGLE_OK) return rc;
    // The arrival counters have to start at zero.  Every call leaves them zero, but the array
    // is shared by all calls on this GPU and outlives them, so they are cleared here as well:
    // a call that was cut short cannot poison the next one.
    const int n = L.ranges < MAX_RANGES ? L.ranges : MAX_RANGES;
    hipLaunchKernelGGL(zero_u32_kernel, dim3((n + 255) / 256), dim3(256), 0, st, static_cast<unsigned*>(ws), n);
  }
  return run(x, wq, scales, biases, bias, out, M, N, K, L, 0, ws, ws_bytes, st);
}

EAGLE_EXPORT int eagle_qmm_swiglu_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                            const void* biases, const void* bias, void* out,
                                            int M, int N, int K, int group_size, int bits,
                                            void* workspace, size_t workspace_bytes,
                                            eagle_stream_t stream) {
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  int rc = validate(x, wq, scales, biases, bias, out, M, N, K);
  if (rc != EAGLE_OK) return rc;
  if ((N % 32) != 0) return EAGLE_ERR_SHAPE;             // whole (gate, up) tile pairs
  Launch L;
  choose(M, N, K, &L);
  if (L.ranges > N / 32) L.ranges = N / 32;
  L.ranges = balanced_ranges(N / 32, L.ranges);
  rc = validate_launch(M, N, K, L, 2);
  if (rc != EAGLE_OK) return rc;
  return run(x, wq, scales, biases, bias, out, M, N, K, L, 1, workspace, workspace_bytes,
             static_cast<hipStream_t>(stream));
}
