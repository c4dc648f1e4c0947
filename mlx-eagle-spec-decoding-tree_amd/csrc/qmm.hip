// 4-bit (group 64) quantised matmul for M = 1..32 rows of x, gfx950.
//
//   out[m,n] = fp16( sum_k x[m,k] * (s[n,k/64] * q[n,k] + b[n,k/64]) )
//
// Weight layout is the MLX one: wq[N, K/8] uint32, nibble i of a word is element
// 8*word + i; scales/biases [N, K/64] fp16.  (Reference contract:
// qmm_kernel.py:84-164, kernels/progression/simd_no_swizzle_cast.metal.)
//
// Structure: a weight streamer with x resident in LDS.
//
//  * A workgroup owns one K slab (at most 4096 columns for M <= 16, 2048 for M <= 32)
//    and a contiguous range of 16-row weight tiles.  It first copies its slab of x
//    into LDS (element order 0,4,1,5,2,6,3,7 inside every group of eight, matching
//    the nibble pairs below), once; after that the only memory traffic of the main
//    loop is the weight stream, and there is no barrier per K step.
//  * Tiles are processed in rounds of WT tiles; WK waves share a tile and split its
//    K chunks (256 columns each).  Per chunk a lane issues two 128-bit loads: the
//    four lanes that share a row read 64 contiguous bytes per instruction, one full
//    128-byte line per chunk.  PF chunks are kept in flight in a register ring that
//    runs across tile rounds.
//  * Nibbles are expanded in registers with the fp16 magic-number trick
//    ((w & 0x000f000f) | 0x6400 = 1024 + q, (w & 0x00f000f0) | 0x5400 = 64 + q), giving
//    the pairs (q0,q4) (q1,q5) (q2,q6) (q3,q7), scaled with packed fp16 FMAs and fed to
//    v_mfma_f32_16x16x32_f16 as the A operand (rows = output features); the B operand
//    (columns = rows of x) is read from the LDS slab; accumulation is fp32.
//  * The WK partial tiles of a round are added through LDS.  K slabs (blockIdx.y) are
//    added through fp32 partials in a workspace: the last workgroup to arrive sums
//    them in slab order, so results are deterministic.  The partials travel as
//    device-scope relaxed atomics (write-through stores, L2-bypassing loads): no
//    L2 write-back / invalidate fence, which costs microseconds on a multi-XCD part.
#include "common.h"

namespace {

constexpr int CHUNK_K = 256;          // K columns per wave step (4 quantisation groups)
constexpr int MAX_ROW_BLOCKS = EAGLE_QMM_COUNTER_BYTES / 4;
constexpr int MAX_SPLITS = 16;
constexpr int MAX_WAVES = 12;          // per workgroup: 768 threads, up to 170 VGPRs each
constexpr int LDS_BUDGET = 160 * 1024 - 512;

__device__ inline half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// (v & mask) | bits in one VALU op.  The compiler splits the two-literal form into
// v_and + v_or; holding `bits` in a VGPR and `mask` in an SGPR makes it encodable.
__device__ inline uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(bits));
  return r;
}

struct DequantConsts {
  uint32_t magic_lo, magic_hi;   // VGPR copies of 0x64006400 / 0x54005400
};

// 8 nibbles of one packed word -> 8 fp16 weights in the order q0,q4,q1,q5,q2,q6,q3,q7.
__device__ inline half8_t dequant8(uint32_t v, half2_t ss, half2_t bb, const DequantConsts& c) {
  const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
  const half2_t k64 = {(half_t)64.0f, (half_t)64.0f};
  const uint32_t v2 = v >> 8;
  half2_t a0 = as_h2(and_or(v, 0x000f000fu, c.magic_lo)) - k1024;    // 1024 + q  -> q
  half2_t a1 = as_h2(and_or(v, 0x00f000f0u, c.magic_hi)) - k64;      //   64 + q  -> q
  half2_t a2 = as_h2(and_or(v2, 0x000f000fu, c.magic_lo)) - k1024;
  half2_t a3 = as_h2(and_or(v2, 0x00f000f0u, c.magic_hi)) - k64;
  a0 = a0 * ss + bb;
  a1 = a1 * ss + bb;
  a2 = a2 * ss + bb;
  a3 = a3 * ss + bb;
  half8_t r;
  r[0] = a0[0]; r[1] = a0[1]; r[2] = a1[0]; r[3] = a1[1];
  r[4] = a2[0]; r[5] = a2[1]; r[6] = a3[0]; r[7] = a3[1];
  return r;
}

// One chunk of one 16-row tile as held by a lane, exactly as loaded (nothing may be
// computed from these registers before the chunk is consumed, or the wait for it would
// drain the whole prefetch ring): 2 x 32 nibbles of its row.
struct WRegs {
  uint4_t lo, hi;
};

struct Launch {
  int rt;          // 16-row tiles per wave (1 or 2)
  int wt;          // tile slots per round (waves along N)
  int wk;          // waves sharing a tile (each takes a contiguous run of the slab's chunks)
  int splits;      // K slabs (gridDim.y)
  int slab_k;      // columns per slab, multiple of 256
  int row_groups;  // gridDim.x
  int rounds;      // tile rounds per workgroup
  int pf;          // ring depth (4, 5 or 7): the divisor of the run length that wastes least
};

constexpr int SB_ITERS = 4;   // 64 lanes x 4 cover the 16 rows x (<= 16 chunks) of a wave's run

// LDS stride (in 8-byte units) of one row of a wave's scale / bias block: odd, so that the
// 16 rows read by one quarter wave fall into 16 different bank pairs.
__host__ __device__ inline int sb_row_units(int units) { return units | 1; }

// PF = weight chunks in flight per wave (depth of the register ring).
template <int NT, int RT, int PF, bool SLOW_SB>
__global__ __launch_bounds__(768) void qmm_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w,
    const half_t* __restrict__ s, const half_t* __restrict__ b,
    const half_t* __restrict__ bias, half_t* __restrict__ out,
    float* __restrict__ partial, unsigned* __restrict__ counters,
    int M, int N, int K, int WT, int WK, int slab_k, int rounds) {
  constexpr int MP = 16 * NT;                     // padded rows of x
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int nthr = blockDim.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wt = wave % WT;
  const int wk = wave / WT;
  const int r = lane & 15;   // row inside a 16-row tile (A operand) / column m (B operand)
  const int h = lane >> 4;   // which 32-nibble quarter of a 128-nibble half chunk
  const int G = K >> 6;
  const int K8 = K >> 3;
  const int nsplit = gridDim.y;

  const int k0 = blockIdx.y * slab_k;
  const int klen = min(slab_k, K - k0);
  const int nchunks = (klen + CHUNK_K - 1) / CHUNK_K;      // chunks of this slab
  const int cbase = k0 / CHUNK_K;                          // first chunk of the slab in K
  // this wave's contiguous run of chunks inside the slab
  const int U = (slab_k / CHUNK_K + WK - 1) / WK;
  const int c_lo = wk * U;
  const int cpw = max(min(nchunks, c_lo + U) - c_lo, 0);
  const int UP = sb_row_units(U);

  // LDS: [x slab][WK reduction buffer][per-wave scale/bias blocks]
  const int xrow = slab_k * 2 + 16;               // bytes per x row (+16: conflict-free b128)
  unsigned char* red = lds + MP * xrow;
  const int red_bytes = WK > 1 ? (WK - 1) * WT * RT * NT * 1024 : 0;
  const int sb_tile_bytes = 2 * 16 * UP * 8;      // scales then biases of one 16-row tile run
  unsigned char* sbw = red + red_bytes + wave * (RT * sb_tile_bytes);

  const int tiles_per_round = WT * RT;
  const int tile_base = (blockIdx.x * rounds) * tiles_per_round + wt * RT;

  // ---- scales / biases of a round: global -> staging registers -> this wave's LDS block ----
  // Unit (row, u) = the four scales (or biases) of chunk c_lo + u of tile row `row`, 8 bytes.
  // Rows of a tile are adjacent in memory, so a full-K run is one contiguous block.
  uint2_t st_s[RT][SB_ITERS], st_b[RT][SB_ITERS];
  auto load_sb = [&](int round) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int it = 0; it < SB_ITERS; ++it) {
        const int idx = lane + 64 * it;
        const int row = idx / U;
        const int u = idx - row * U;
        const bool ok = round < rounds && idx < 16 * U && u < cpw;
        const int n = min((tile_base + min(round, rounds - 1) * tiles_per_round + rt) * 16 + min(row, 15), N - 1);
        const int c4 = (cbase + c_lo + min(u, max(cpw - 1, 0))) * 4;
        if (SLOW_SB) {
          // fewer than four groups per row, or an odd group count: element-wise
          uint32_t sv[4], bv[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool oki = ok && (c4 + i) < G;
            const size_t off = (size_t)n * G + min(c4 + i, G - 1);
            sv[i] = oki ? (uint32_t) * reinterpret_cast<const uint16_t*>(s + off) : 0u;
            bv[i] = oki ? (uint32_t) * reinterpret_cast<const uint16_t*>(b + off) : 0u;
          }
          st_s[rt][it] = uint2_t{sv[0] | (sv[1] << 16), sv[2] | (sv[3] << 16)};
          st_b[rt][it] = uint2_t{bv[0] | (bv[1] << 16), bv[2] | (bv[3] << 16)};
        } else {
          // A last chunk with fewer than four groups reads the row's last four groups
          // instead (in range); compute() shifts them into place.
          const size_t off = (size_t)n * G + min(c4, G - 4);
#ifdef EAGLE_DBG_NOSB
          st_s[rt][it] = uint2_t{(uint32_t)off, 0u}; st_b[rt][it] = uint2_t{0u, (uint32_t)n};
#else
          st_s[rt][it] = *reinterpret_cast<const uint2_t*>(s + off);   // unconditional, see load_w
          st_b[rt][it] = *reinterpret_cast<const uint2_t*>(b + off);
#endif
          (void)ok;
        }
      }
  };
  auto commit_sb = [&]() {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int it = 0; it < SB_ITERS; ++it) {
        const int idx = lane + 64 * it;
        const int row = idx / U;
        const int u = idx - row * U;
        if (idx < 16 * U) {
          unsigned char* dst = sbw + rt * sb_tile_bytes + (row * UP + u) * 8;
          *reinterpret_cast<uint2_t*>(dst) = st_s[rt][it];
          *reinterpret_cast<uint2_t*>(dst + 16 * UP * 8) = st_b[rt][it];
        }
      }
  };

  const uint32_t gsel = (h & 2) ? 0x03020302u : 0x01000100u;   // byte selector of group h/2
  DequantConsts dq;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(dq.magic_lo));
  asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(dq.magic_hi));

  // item (round, j): chunk c_lo + j of the slab, for the RT tiles of this wave.  The lane
  // reads nibbles 32h..32h+31 (group 4c + h/2) and 128+32h.. (group 4c + 2 + h/2) of it.
  // Loads are unconditional: a conditional load makes the compiler fall back to waiting
  // for every outstanding load.  Out-of-range rounds, rows, chunks and groups are clamped to
  // an in-range address instead; what they fetch is multiplied by the zeros that pad x in
  // LDS (columns >= K) or never consumed (dummy items, rows >= N).
  auto load_w = [&](int round, int j, WRegs (&dst)[RT]) {
    const int c = cbase + c_lo + j;
    const int col = c * 32 + h * 4;                       // in 32-bit words, 4 per load
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int rr = min(round, rounds - 1);
      const int n = min((tile_base + rr * tiles_per_round + rt) * 16 + r, N - 1);
      const uint32_t* row = w + (size_t)n * K8;
#ifdef EAGLE_DBG_NOW
      dst[rt].lo = uint4_t{(uint32_t)n, 0, 0, 0}; dst[rt].hi = uint4_t{0, 0, 0, (uint32_t)col}; (void)row;
#else
      dst[rt].lo = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(row + min(col, K8 - 4)));
      dst[rt].hi = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(row + min(col + 16, K8 - 4)));
#endif
    }
  };

  float4_t acc[RT][NT];
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](const WRegs (&cur)[RT], int j) {
    // B operand of step t: 8 halves of x row m = 16 nt + r at slab column
    // 256 (c_lo + j) + 32h + 8t (t < 4) or + 128 + 32h + 8(t-4)
    const unsigned char* xb = lds + r * xrow + (c_lo + j) * (CHUNK_K * 2) + h * 64;
    // the lane's groups are h/2 (first half chunk) and 2 + h/2: broadcast that half of
    // the {g0,g1} / {g2,g3} pairs into both halves of a register
    half2_t ss[RT][2], bb[RT][2];
    const int c4 = (cbase + c_lo + j) * 4;
    const int shift = SLOW_SB ? 0 : 16 * (c4 - min(c4, G - 4));   // tail chunk: see load_sb
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const unsigned char* sp = sbw + rt * sb_tile_bytes + (r * UP + j) * 8;
      const uint2_t s4 = *reinterpret_cast<const uint2_t*>(sp);
      const uint2_t b4 = *reinterpret_cast<const uint2_t*>(sp + 16 * UP * 8);
      uint32_t s01 = s4[0], s23 = s4[1], b01 = b4[0], b23 = b4[1];
      if (shift) {
        const uint64_t sv = (((uint64_t)s23 << 32) | s01) >> shift;
        const uint64_t bv = (((uint64_t)b23 << 32) | b01) >> shift;
        s01 = (uint32_t)sv; s23 = (uint32_t)(sv >> 32);
        b01 = (uint32_t)bv; b23 = (uint32_t)(bv >> 32);
      }
      ss[rt][0] = as_h2(__builtin_amdgcn_perm(s01, s01, gsel));
      bb[rt][0] = as_h2(__builtin_amdgcn_perm(b01, b01, gsel));
      ss[rt][1] = as_h2(__builtin_amdgcn_perm(s23, s23, gsel));
      bb[rt][1] = as_h2(__builtin_amdgcn_perm(b23, b23, gsel));
    }
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      half8_t bx[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        bx[nt] = *reinterpret_cast<const half8_t*>(xb + nt * 16 * xrow + (t >> 2) * 256 + (t & 3) * 16);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const uint32_t word = (t < 4) ? cur[rt].lo[t & 3] : cur[rt].hi[t & 3];
        const half8_t a = dequant8(word, ss[rt][t >> 2], bb[rt][t >> 2], dq);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx[nt], acc[rt][nt], 0, 0, 0);
      }
    }
  };

  // End of a round: add the WK partial tiles, combine K slabs, store.
  auto finish_round = [&](int round) {
    if (WK > 1) {
      float4_t* rb = reinterpret_cast<float4_t*>(red);
      __syncthreads();                 // previous round's readers are done with `red`
      if (wk > 0) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            rb[((((wk - 1) * WT + wt) * RT + rt) * NT + nt) * 64 + lane] = acc[rt][nt];
      }
      __syncthreads();
      if (wk == 0) {
        for (int k2 = 1; k2 < WK; ++k2)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
              acc[rt][nt] += rb[((((k2 - 1) * WT + wt) * RT + rt) * NT + nt) * 64 + lane];
      }
    }
    const bool owner = wk == 0;
    bool write_out = owner;
    if (nsplit > 1) {
      const int rblock = blockIdx.x * rounds + round;       // row block of this round
      const int per_blk = WT * RT * NT * 64;                // float4 per (row block, slab)
      float* pbase = partial + ((size_t)rblock * nsplit) * per_blk * 4;
      if (owner) {
        float* mine = pbase + (size_t)blockIdx.y * per_blk * 4;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              __hip_atomic_store(mine + ((((wt * RT + rt) * NT + nt) * 64 + lane) << 2) + i,
                                 acc[rt][nt][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's partial stores are done
      __syncthreads();
      if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&counters[rblock], 1u, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (unsigned)(nsplit - 1));
      }
      __syncthreads();
      const bool last = s_last != 0;
      write_out = owner && last;
      if (write_out) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            float4_t sum = float4_t{0.f, 0.f, 0.f, 0.f};
            for (int sp = 0; sp < nsplit; ++sp) {
              const float* src = pbase + (size_t)sp * per_blk * 4 +
                                 ((((wt * RT + rt) * NT + nt) * 64 + lane) << 2);
#pragma unroll
              for (int i = 0; i < 4; ++i)
                sum[i] += __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            acc[rt][nt] = sum;
          }
      }
      if (last && tid == 0)
        __hip_atomic_store(&counters[rblock], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // lane holds out[m = 16 nt + r][n = tile*16 + 4 h + i], i = 0..3
    if (write_out) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int n0 = (tile_base + round * tiles_per_round + rt) * 16 + 4 * h;
        if (n0 >= N) continue;   // N % 8 == 0, so a group of four is all in or all out
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int m = nt * 16 + r;
          if (m >= M) continue;
          half4_t o;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            half_t v = (half_t)acc[rt][nt][i];
            if (bias) v = (half_t)((float)v + (float)bias[n0 + i]);
            o[i] = v;
          }
          *reinterpret_cast<half4_t*>(out + (size_t)m * N + n0) = o;
        }
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
    // Stores and loads retire out of order with respect to each other, so a counted wait
    // on the weight ring is only exact while no store is pending: drain here, once per
    // round, instead of at every chunk.  (0x0F70 = vmcnt(0), other counters untouched.)
    __builtin_amdgcn_s_waitcnt(0x0F70);
  };

  // ---- prologue: first loads in flight, then the x slab ---------------------------------
  // Every wave walks UPAD = U rounded up to a multiple of PF items per round, so that the
  // ring slot of an item is a compile-time constant; items past its real run are dummies
  // (no load, no compute).
  const int UPAD = (U + PF - 1) / PF * PF;
  // Order matters: the x loads go out first and in one batch where possible (they sit on
  // the critical path to the first barrier), the weight ring next; waiting for x then
  // leaves the younger ring loads in flight.
  load_sb(0);
  {
    constexpr int XB = 12;
    const int vec_row = slab_k >> 3;
    const int total = MP * vec_row;
    for (int v0 = tid; v0 < total; v0 += nthr * XB) {
      half8_t a[XB];
#pragma unroll
      for (int i = 0; i < XB; ++i) {
        // always load from an in-range address and zero afterwards: no branch, so the
        // XB loads are in flight together
        const int v = v0 + i * nthr;
        const int row = v / vec_row;
        const int c8 = v - row * vec_row;
        const int k = k0 + c8 * 8;
        const bool ok = v < total && row < M && k < K;
        const half8_t ld = *reinterpret_cast<const half8_t*>(
            x + (size_t)min(row, M - 1) * K + min(k, K - 8));
        a[i] = ok ? ld : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
      for (int i = 0; i < XB; ++i) {
        const int v = v0 + i * nthr;
        const int row = v / vec_row;
        const int c8 = v - row * vec_row;
        half8_t p;   // element order matching dequant8: 0,4,1,5,2,6,3,7
        p[0] = a[i][0]; p[1] = a[i][4]; p[2] = a[i][1]; p[3] = a[i][5];
        p[4] = a[i][2]; p[5] = a[i][6]; p[6] = a[i][3]; p[7] = a[i][7];
        if (v < total) *reinterpret_cast<half8_t*>(lds + row * xrow + c8 * 16) = p;
      }
    }
  }
  WRegs ring[PF][RT];
#pragma unroll
  for (int p = 0; p < PF; ++p) load_w(0, p, ring[p]);
  commit_sb();
  load_sb(1);
  __syncthreads();                      // the x slab is in LDS

  // ---- main loop -------------------------------------------------------------------------
  // The chunk loop is free of stores and of round bookkeeping, so the counted waits on the
  // ring stay exact; the ring runs across rounds (the last PF items of a round already
  // load the first PF of the next).
  for (int round = 0; round < rounds; ++round) {
    for (int jb = 0; jb < UPAD; jb += PF) {
#pragma unroll
      for (int p = 0; p < PF; ++p) {
        const int j = jb + p;
        if (j < cpw) {
#ifdef EAGLE_DBG_NOCOMP
          acc[0][0][0] += __builtin_bit_cast(float, ring[p][0].lo[0] ^ ring[p][0].hi[3]);
#else
          compute(ring[p], j);
#endif
        }
        int nj = j + PF, nr = round;
        if (nj >= UPAD) { nj -= UPAD; ++nr; }
        load_w(nr, nj, ring[p]);
      }
    }
#ifndef EAGLE_DBG_NOSTORE
    finish_round(round);
#endif
    commit_sb();               // staged while the round that just ended was running
    load_sb(round + 2);
  }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
// Ring depth for a run of `units` chunks: the depth whose multiple overshoots the run least
// (the overshoot only costs empty loop iterations); deeper wins ties.
int pick_pf(int units) {
  int best = 7, best_waste = 1 << 30;
  const int cands[3] = {7, 5, 4};
  for (int pf : cands) {
    const int waste = (units + pf - 1) / pf * pf - units;
    if (waste < best_waste) { best = pf; best_waste = waste; }
  }
  return best;
}

int lds_bytes(int mp, const Launch& L) {
  const int nt = mp / 16;
  const int xs = mp * (L.slab_k * 2 + 16);
  const int red = L.wk > 1 ? (L.wk - 1) * L.wt * L.rt * nt * 1024 : 0;
  const int units = (L.slab_k / CHUNK_K + L.wk - 1) / L.wk;
  const int sb = L.wt * L.wk * L.rt * 2 * 16 * sb_row_units(units) * 8;
  return xs + red + sb;
}

int validate_launch(int M, int N, int K, const Launch& L) {
  const int mp = M <= 16 ? 16 : 32;
  if (L.rt != 1 || L.wt < 1 || L.wk < 1 || L.wt * L.wk > MAX_WAVES) return EAGLE_ERR_SHAPE;
  if (L.pf != 4 && L.pf != 5 && L.pf != 7) return EAGLE_ERR_SHAPE;
  if (L.splits < 1 || L.splits > MAX_SPLITS || L.slab_k < CHUNK_K || (L.slab_k % CHUNK_K) != 0)
    return EAGLE_ERR_SHAPE;
  if ((long)L.slab_k * L.splits < K || (long)L.slab_k * (L.splits - 1) >= K) return EAGLE_ERR_SHAPE;
  const int units = (L.slab_k / CHUNK_K + L.wk - 1) / L.wk;
  if (units > 16) return EAGLE_ERR_SHAPE;            // a wave's run must fit its staging registers
  if (L.row_groups < 1 || L.rounds < 1) return EAGLE_ERR_SHAPE;
  const long tiles = (N + 15) / 16;
  if ((long)L.row_groups * L.rounds * L.wt * L.rt < tiles) return EAGLE_ERR_SHAPE;
  if (lds_bytes(mp, L) > LDS_BUDGET) return EAGLE_ERR_SHAPE;
  if (L.splits > 1 && (long)L.row_groups * L.rounds > MAX_ROW_BLOCKS) return EAGLE_ERR_SHAPE;
  return EAGLE_OK;
}

size_t partial_bytes(int M, const Launch& L) {
  if (L.splits <= 1) return 0;
  const size_t mp = M <= 16 ? 16 : 32;
  return (size_t)L.row_groups * L.rounds * L.splits * L.wt * L.rt * 16 * mp * sizeof(float);
}

// Launch shape.  K slabs only as far as LDS capacity forces them (every extra slab costs
// a partial-sum round trip): the x slab plus the per-wave scale/bias blocks must leave room
// for at least 12 waves.  One workgroup per compute unit when the slab is large, up to four
// when it is small.  As many waves along N as the tile count can feed; the rest of the
// parallelism comes from splitting a tile's chunk run over waves.
void choose(int M, int N, int K, Launch* out) {
  const int mp = M <= 16 ? 16 : 32;
  const int tiles = (N + 15) / 16;
  Launch L;
  L.rt = 1;
  int waves = 4, wg_per_cu = 1;
  bool found = false;
  for (L.splits = 1; L.splits <= MAX_SPLITS && !found; ++L.splits) {
    L.slab_k = ((K + L.splits - 1) / L.splits + CHUNK_K - 1) / CHUNK_K * CHUNK_K;
    const int chunks = L.slab_k / CHUNK_K;
    if (chunks > 16) continue;                               // staging registers hold 16 chunks
    const int x_lds = mp * (L.slab_k * 2 + 16);
    const int sb_wave = 2 * 16 * sb_row_units(chunks) * 8;
    const bool last_try = L.splits == MAX_SPLITS || L.slab_k == CHUNK_K;
    for (int wg = 4; wg >= 1 && !found; --wg) {
      int w = (LDS_BUDGET / wg - 1024 - x_lds) / sb_wave;
      if (w > 16 / wg) w = 16 / wg;
      if (w > MAX_WAVES) w = MAX_WAVES;
      w = w / 4 * 4;
      if (w >= 4 && (wg * w >= 12 || (last_try && wg == 1))) {
        waves = w;
        wg_per_cu = wg;
        found = true;
      }
    }
    if (found) break;
  }
  L.splits = (K + L.slab_k - 1) / L.slab_k;
  const int chunks = L.slab_k / CHUNK_K;
  const int nchunks_last = (K - L.slab_k * (L.splits - 1) + CHUNK_K - 1) / CHUNK_K;
  int groups = (256 * wg_per_cu) / L.splits;
  if (groups < 1) groups = 1;
  if (groups > tiles) groups = tiles;
  const int tiles_per_group = (tiles + groups - 1) / groups;
  if (tiles_per_group >= waves) {
    L.wk = 1;
    L.rounds = (tiles_per_group + waves - 1) / waves;
    L.wt = (tiles_per_group + L.rounds - 1) / L.rounds;      // even out the rounds
  } else {
    L.wt = tiles_per_group;
    L.wk = waves / L.wt;
    if (L.wk > chunks) L.wk = chunks;
    // every wave should own at least one chunk of the (shorter) last slab
    while (L.wk > 1 && ((chunks + L.wk - 1) / L.wk) * (L.wk - 1) >= nchunks_last) --L.wk;
    L.rounds = 1;
  }
  L.row_groups = (tiles + L.rounds * L.wt - 1) / (L.rounds * L.wt);
  L.pf = pick_pf((chunks + L.wk - 1) / L.wk);
  *out = L;
}

template <int NT, int PF, bool SLOW_SB>
int launch(const void* x, const uint32_t* wq, const void* s, const void* b, const void* bias,
           void* out, float* partial, unsigned* counters, int M, int N, int K, const Launch& L,
           hipStream_t stream) {
  const int lds = lds_bytes(16 * NT, L);
  static bool attr_set = false;   // more than 64 KB of LDS needs an explicit opt-in, once
  if (lds > 65536 && !attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_w4g64_kernel<NT, 1, PF, SLOW_SB>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BUDGET) != hipSuccess)
      return EAGLE_ERR_HIP;
    attr_set = true;
  }
  hipLaunchKernelGGL((qmm_w4g64_kernel<NT, 1, PF, SLOW_SB>), dim3(L.row_groups, L.splits),
                     dim3(64 * L.wt * L.wk), lds, stream, (const half_t*)x, wq,
                     (const half_t*)s, (const half_t*)b, (const half_t*)bias, (half_t*)out,
                     partial, counters, M, N, K, L.wt, L.wk, L.slab_k, L.rounds);
  return eagle_launch_status();
}

int validate(const void* x, const uint32_t* wq, const void* s, const void* b, const void* bias,
             void* out, int M, int N, int K) {
  if (!x || !wq || !s || !b || !out) return EAGLE_ERR_NULL;
  if (M < 1 || M > EAGLE_MAX_M || N < 8 || (N % 8) != 0 || K < 64 || (K % 64) != 0)
    return EAGLE_ERR_SHAPE;
  const int slab_max = M <= 16 ? 4096 : 2048;
  if (K > slab_max * MAX_SPLITS) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(out) ||
      (reinterpret_cast<uintptr_t>(s) & 1u) || (reinterpret_cast<uintptr_t>(b) & 1u) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  return EAGLE_OK;
}

int run(const void* x, const uint32_t* wq, const void* scales, const void* biases,
        const void* bias, void* out, int M, int N, int K, const Launch& L, void* workspace,
        size_t workspace_bytes, hipStream_t st) {
  float* partial = nullptr;
  unsigned* counters = nullptr;
  if (L.splits > 1) {
    if (!workspace || !eagle_aligned16(workspace) ||
        workspace_bytes < (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, L))
      return EAGLE_ERR_WORKSPACE;
    counters = reinterpret_cast<unsigned*>(workspace);
    partial = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) +
                                       EAGLE_QMM_COUNTER_BYTES);
  }
  // rows with fewer than four groups, or an odd group count (unaligned 8-byte reads),
  // fetch scales and biases one by one
  const int G = K / 64;
  const bool slow = G < 4 || (G & 1);
#define EAGLE_QMM_GO(NT_, PF_)                                                               \
  return slow ? launch<NT_, PF_, true>(x, wq, scales, biases, bias, out, partial, counters, \
                                       M, N, K, L, st)                                      \
              : launch<NT_, PF_, false>(x, wq, scales, biases, bias, out, partial, counters, \
                                        M, N, K, L, st)
  if (M <= 16) {
    if (L.pf == 7) EAGLE_QMM_GO(1, 7);
    if (L.pf == 5) EAGLE_QMM_GO(1, 5);
    EAGLE_QMM_GO(1, 4);
  }
  if (L.pf == 7) EAGLE_QMM_GO(2, 7);
  if (L.pf == 5) EAGLE_QMM_GO(2, 5);
  EAGLE_QMM_GO(2, 4);
#undef EAGLE_QMM_GO
}

}  // namespace

EAGLE_EXPORT size_t eagle_qmm_workspace_bytes(int M, int N, int K) {
  if (M < 1 || M > EAGLE_MAX_M || N < 1 || K < 64) return 0;
  Launch L;
  choose(M, N, K, &L);
  return (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, L);
}

EAGLE_EXPORT size_t eagle_qmm_workspace_bytes_tuned(int M, int rt, int wt, int wk, int splits,
                                                    int row_groups, int rounds) {
  if (M < 1 || rt < 1 || wt < 1 || wk < 1 || splits < 1 || row_groups < 1 || rounds < 1) return 0;
  Launch L{rt, wt, wk, splits, 0, row_groups, rounds, 4};
  return (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(M, L);
}

EAGLE_EXPORT int eagle_qmm_plan(int M, int N, int K, int* plan7) {
  if (!plan7) return EAGLE_ERR_NULL;
  if (M < 1 || M > EAGLE_MAX_M || N < 8 || K < 64 || (K % 64) != 0) return EAGLE_ERR_SHAPE;
  Launch L;
  choose(M, N, K, &L);
  plan7[0] = L.rt; plan7[1] = L.wt; plan7[2] = L.wk; plan7[3] = L.splits;
  plan7[4] = L.slab_k; plan7[5] = L.row_groups; plan7[6] = L.rounds;
  return EAGLE_OK;
}

EAGLE_EXPORT int eagle_qmm_w4g64_f16_tuned(const void* x, const uint32_t* wq, const void* scales,
                                           const void* biases, const void* bias, void* out, int M,
                                           int N, int K, int rt, int wt, int wk, int splits,
                                           int slab_k, int row_groups, int rounds, void* workspace,
                                           size_t workspace_bytes, eagle_stream_t stream) {
  int rc = validate(x, wq, scales, biases, bias, out, M, N, K);
  if (rc != EAGLE_OK) return rc;
  Launch L{rt, wt, wk, splits, slab_k, row_groups, rounds, 0};
  L.pf = pick_pf((slab_k / CHUNK_K + (wk > 0 ? wk : 1) - 1) / (wk > 0 ? wk : 1));
  rc = validate_launch(M, N, K, L);
  if (rc != EAGLE_OK) return rc;
  return run(x, wq, scales, biases, bias, out, M, N, K, L, workspace, workspace_bytes,
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
  return run(x, wq, scales, biases, bias, out, M, N, K, L, workspace, workspace_bytes,
             static_cast<hipStream_t>(stream));
}
