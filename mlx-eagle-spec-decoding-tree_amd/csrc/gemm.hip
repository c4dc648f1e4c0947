// 4-bit group-64 quantised matmul for many rows (the prompt pass, mlx_eagle.py:522-533 through
// the QuantizedLinear layers of mlx_llama.py): out[M,N] = fp16( x[M,K] . (s*q + b)[N,K]^T ).
//
// With hundreds of rows the product is bound by the matrix cores, not by the weight stream, so
// this is a tiled GEMM: a workgroup of four waves side by side along the weight rows owns a
// 64 x 128, 128 x 128 or 128 x 256 output block (x rows x weight rows), each wave all x rows of
// the block as v_mfma_f32_32x32x16_f16 tiles (weights are the A operand: an accumulator lane
// then holds one output row and four consecutive columns per register group).  Per 64-wide K
// step (one quantisation group):
//   * the x block goes through LDS (double buffered, one barrier per step), loaded one or two
//     steps ahead into registers, a whole 128-byte row of the step per eight lanes;
//   * every lane loads the 16 bytes (four packed words = 32 weights) of its weight row that its
//     half of the MFMA K range needs, two steps ahead, and expands them in registers:
//     a shift and v_and_or_b32 make the fp16 pair (16 + q_i, 16 + q_{i+4}); one packed fp16
//     fma with (s, b - 16 s) gives the weights in fp16, as the reference kernels hold them.
//     That yields the eight weights of a word in the order q0 q4 q1 q5 q2 q6 q3 q7; x is stored
//     to LDS in the same order within every group of eight, so both MFMA operands agree on
//     which K index sits where.  The expanded word j of a step is replaced by the next step's
//     as soon as this step's matrix instructions have read it (one register set, which lets
//     two workgroups share a compute unit with the 128 x 256 block);
//   * the output tile of a wave leaves through LDS as whole rows.
// Measured for 512 x 28672 x 4096 (s_memtime / s_memrealtime inside the kernel): the core clock
// is 1.55 - 1.85 GHz while this kernel runs (a loop of matrix instructions alone sustains 2.1 - 2.4
// PFLOP/s on the same box), a workgroup alone on a compute unit needs 1900 clocks per step for
// 1024 clocks of matrix instructions, two together 1330 each; 448 workgroups on 512 places leave
// a quarter of the compute units with one workgroup, which ends 25 % before the others.  Blocks
// of 128 x 512 and 256 x 256 (half the LDS reads, or half the expansions, per matrix instruction;
// 512 registers, one workgroup per compute unit) were 3 - 5 % faster on that shape and half as
// fast on the narrow ones, and are not built.  The narrow shapes (N = 4096: one 64 x 128 block per
// compute unit) run two groups of four waves per workgroup, each over half of K (+5 %); loading
// the packed weights by whole 128-byte lines (timing only, results wrong) is worth 0 - 7 %.
// fp32 accumulation, one fp16 rounding, optional fp16 bias added after the rounding.
#include "common.h"

namespace {

constexpr int BK = 64;
constexpr long GEMM_SPLIT_WGS = 384;        // two K groups per workgroup up to this many workgroups
constexpr long NUM_CU = 256;
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
// Every nibble is moved to the top four mantissa bits of 16.0 (0x4c00), where one step is 1:
// the fp16 pair is (16 + q_i, 16 + q_{i+4}) and one packed fma with (s, b - 16 s) gives the
// weights.  (Nibbles left in the low mantissa bits would need an offset of 1024 s, which does
// not leave b enough bits; with 16 s the rounding of b - 16 s is below 1e-3 of a weight.)
__device__ inline half8_t dequant_word(uint32_t w, half2_t s2, half2_t b16) {
  union { uint32_t u; half2_t h; } c[4];
  c[0].u = and_or(w << 6, 0x03c003c0u, 0x4c004c00u);
  c[1].u = and_or(w << 2, 0x03c003c0u, 0x4c004c00u);
  c[2].u = and_or(w >> 2, 0x03c003c0u, 0x4c004c00u);
  c[3].u = and_or(w >> 6, 0x03c003c0u, 0x4c004c00u);
  half8_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t v = __builtin_elementwise_fma(c[i].h, s2, b16);
    o[2 * i] = v[0];
    o[2 * i + 1] = v[1];
  }
  return o;
}

// The same with the offset taken off first: (16 + q) - 24 = q - 8 exactly, then one packed fma
// with (s, b + 8 s).  For weights quantised the usual way b is close to -8 s, so b + 8 s is
// small and its rounding no longer matters (with b - 16 s, about 24 s in size, that rounding is
// 0.15 % of a weight, and it is the same for all 64 weights of a group).  One packed add more
// per pair: for the kernel below, which is not bound by the expansion.
__device__ inline half8_t dequant_word_centred(uint32_t w, half2_t s2, half2_t b8) {
  union { uint32_t u; half2_t h; } c[4];
  c[0].u = and_or(w << 6, 0x03c003c0u, 0x4c004c00u);
  c[1].u = and_or(w << 2, 0x03c003c0u, 0x4c004c00u);
  c[2].u = and_or(w >> 2, 0x03c003c0u, 0x4c004c00u);
  c[3].u = and_or(w >> 6, 0x03c003c0u, 0x4c004c00u);
  const half2_t off = half2_t{(half_t)24.f, (half_t)24.f};
  half8_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t v = __builtin_elementwise_fma(c[i].h - off, s2, b8);
    o[2 * i] = v[0];
    o[2 * i + 1] = v[1];
  }
  return o;
}

// Through fp16 subnormals: a masked nibble pair left at mantissa bits 4..7 is (q_i, q_j) * 2^-20
// exactly, and one packed fma with (s * 2^20, b) gives fp16(s*q + b) with a single rounding and
// no offset: three shifts, four masks and four fmas per packed word.  |s| * 2^20 has to stay
// inside fp16: |s| < 0.0624 (beyond it the product is inf / NaN).
__device__ inline half8_t dequant_word_sub(uint32_t w, half2_t s20, half2_t b2) {
  union { uint32_t u; half2_t h; } c[4];
  c[0].u = (w << 4) & 0x00f000f0u;
  c[1].u = w & 0x00f000f0u;
  c[2].u = (w >> 4) & 0x00f000f0u;
  c[3].u = (w >> 8) & 0x00f000f0u;
  half8_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t v = __builtin_elementwise_fma(c[i].h, s20, b2);
    o[2 * i] = v[0];
    o[2 * i + 1] = v[1];
  }
  return o;
}

// MT = 32-row x tiles per wave: 2 (128-row blocks) or 4 (256-row blocks: twice the matrix work
// per expanded weight and per byte read from LDS).
template <int E>
struct StepIndex {
  static constexpr int value = E;
};

// SBW = groups per fetch of scales and biases (1, 2, 4 or 8; K is a multiple of 64 * SBW): one
// fetch per SBW K steps instead of one 2-byte load per row and step (the loads of one
// instruction go to 32 or 64 different cache lines either way, and the rate of such requests,
// not their bytes, is what the kernel runs up against).
// KGRP = groups of four waves per workgroup (1 or 2).  With two, each group works through its
// own half of K with its own x buffers (one barrier serves both) and the halves are added
// through LDS at the end: for shapes that give a compute unit a single workgroup, whose four
// waves would otherwise have nothing to overlap their waits with.
// SWI: the weight rows are gate and up rows interleaved in 16-row tiles (rows 0..15 of a 32-row
// matrix tile gate, 16..31 the matching up rows: the same accumulator lane holds both); the
// result is silu(g) * u, [M, N / 2].
template <int NTW, int MT, int SBW, int KGRP = 1, bool SWI = false>
__global__ __launch_bounds__(256 * KGRP, (KGRP == 1 ? 2 : 1)) void qmm_gemm_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w, const half_t* __restrict__ s,
    const half_t* __restrict__ b, const half_t* __restrict__ bias, half_t* __restrict__ out, int M,
    int N, int K) {
  // NTW = 32-row weight tiles per wave (1 or 2); the four waves sit side by side along the
  // weight rows, each over all x rows of the block: no weight row is loaded or expanded twice,
  // and with NTW = 2 every x operand read from LDS serves two matrix instructions
  constexpr int WN = 4;                      // waves along the weight rows (side by side)
  constexpr int WM = 1;                      // waves along the x rows
  constexpr int BN = 32 * NTW * WN;          // weight rows per workgroup (128 or 256)
  constexpr int BMT = 32 * MT * WM;          // rows of x per workgroup
  constexpr int TPR = 256 / BMT;             // threads per x row in the block load (2 or 1)
  constexpr int PP = 8 / TPR;                // 16-byte pieces per thread
  extern __shared__ __attribute__((aligned(16))) half_t xs_all[];
  const int grp = KGRP == 1 ? 0 : (int)(threadIdx.x >> 8);    // which part of K this group of waves takes
  half_t* xs[2] = {xs_all + grp * (2 * BMT * XS), xs_all + grp * (2 * BMT * XS) + BMT * XS};
  const int tid = threadIdx.x & 255;
  const int wave = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int wn = wave % WN, wm = wave / WN;
  const int n0 = blockIdx.x * BN + wn * 32 * NTW;
  const int m0 = blockIdx.y * BMT;
  const int KW = K >> 3;                    // packed words per weight row
  const int KG = K >> 6;                    // groups per weight row
  const int steps = K / BK / KGRP;          // of this group
  const int kbase = grp * steps * BK;       // its first column
  x += kbase;
  w += kbase >> 3;
  s += kbase >> 6;
  b += kbase >> 6;

  // thread (xr, xc) moves the 16 bytes at column 8 xc of rows xr + 32 g: a load instruction of a
  // wave covers eight whole 128-byte rows of the step (the rate of cache lines touched, not
  // bytes, bounds the loads of this kernel)
  const int xr = tid >> 3, xc = tid & 7;
  uint32_t xo[PP];                          // element offsets (the host checks M * K < 2^31)
#pragma unroll
  for (int g = 0; g < PP; ++g) {
    int xrow = m0 + xr + 32 * g;
    if (xrow > M - 1) xrow = M - 1;         // rows past the end are never stored
    xo[g] = (uint32_t)xrow * (uint32_t)K + xc * 8;
  }
  int nrow[NTW];
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt) {
    nrow[nt] = n0 + nt * 32 + ql;
    if (nrow[nt] > N - 1) nrow[nt] = N - 1;
  }

  // x is requested one step ahead, or two with the small blocks: their few matrix instructions
  // per step do not cover the latency of that load, and a step cannot be shorter than the lead
  constexpr int XD = MT <= 2 ? 2 : 1;
  half8_t xreg[XD][PP];
  // packed weights: two steps in flight, four with the small blocks (where the unrolled loop
  // makes the register set of a step a constant), for the same reason
  constexpr int WD = (MT <= 2 && SBW >= 4) ? 4 : 2;
  uint4_t wreg[WD][NTW];
  constexpr bool SBV = SBW > 1;
  typedef half_t sbvec_t __attribute__((ext_vector_type(SBV ? SBW : 2)));
  half_t sreg[2][NTW], breg[2][NTW];        // SBW = 1: scale and bias of those steps
  sbvec_t s8[2][NTW], b8[2][NTW];           // SBW > 1: of this chunk of SBW steps and of the next
  half8_t af[NTW][4];                       // expanded weights of this step; word j is replaced by the next
                                            // step's as soon as this step's matrix instructions have read it
  auto fetch_x = [&](int ks, int set) {
#pragma unroll
    for (int g = 0; g < PP; ++g) xreg[set][g] = *reinterpret_cast<const half8_t*>(x + (xo[g] + (uint32_t)(ks * BK)));
  };
  auto fetch_w = [&](int ks, int p) {
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      wreg[p][nt] = *reinterpret_cast<const uint4_t*>(w + (long)nrow[nt] * KW + ks * 8 + hb * 4);
      if (!SBV) {
        sreg[p][nt] = s[(long)nrow[nt] * KG + ks];
        breg[p][nt] = b[(long)nrow[nt] * KG + ks];
      }
    }
  };
  auto fetch_sb = [&](int chunk, int q) {
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      s8[q][nt] = *reinterpret_cast<const sbvec_t*>(s + (long)nrow[nt] * KG + chunk * SBW);
      b8[q][nt] = *reinterpret_cast<const sbvec_t*>(b + (long)nrow[nt] * KG + chunk * SBW);
    }
  };
  auto stash = [&](int buf) {                // x of a step travels in register set (step % XD)
#pragma unroll
    for (int g = 0; g < PP; ++g)
      *reinterpret_cast<half8_t*>(&xs[buf][(xr + 32 * g) * XS + xc * 8]) = permute8(xreg[buf % XD][g]);
  };
  // word j of the weight tiles of register set p; e = index of their step within the chunk of
  // SBW (SBW = first step of the next chunk)
  auto expand = [&](int j, int e) {
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      const half_t sc = SBV ? s8[e / SBW][nt][e % SBW] : sreg[e & 1][nt];
      const half_t bi = SBV ? b8[e / SBW][nt][e % SBW] : breg[e & 1][nt];
      const half_t b16 = (half_t)((float)bi - 16.f * (float)sc);
      af[nt][j] = dequant_word(wreg[e % WD][nt][j], half2_t{sc, sc}, half2_t{b16, b16});
    }
  };

  float16_t acc[NTW][MT];                   // [weight tile][x tile]
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;

  const int chunks = steps / SBW;
  fetch_x(0, 0);
  if (XD == 2) fetch_x(steps > 1 ? 1 : 0, 1);
#pragma unroll
  for (int i = 0; i < WD; ++i) fetch_w(i < steps ? i : steps - 1, i);
  if (SBV) {
    fetch_sb(0, 0);
    fetch_sb(chunks > 1 ? 1 : 0, 1);
  }
  stash(0);
#pragma unroll
  for (int j = 0; j < 4; ++j) expand(j, 0);
  __syncthreads();

  // One K step, p = ks & 1: LDS buffer p holds x of this step and af its expanded weights;
  // register set p ^ 1 holds the packed weights and the x of the next step (the weights are
  // expanded into af word by word behind this step's matrix instructions, the x goes to LDS at
  // its end); set p is free for the loads of step ks + 2.  Loaded
  // values are used where they were loaded (a copy of a register with a load in flight would
  // wait for the load), and the loads are issued first (left alone, the scheduler sinks them
  // to the end of the step, where the in-order counter waits for them at once).
  auto body = [&](int ks, auto E) {
    constexpr int e = decltype(E)::value;   // step within its chunk (SBW > 1) / parity of the step
    constexpr int p = e & 1;
    fetch_x(ks + XD < steps ? ks + XD : steps - 1, p % XD);   // that set's x is in LDS already
    fetch_w(ks + WD < steps ? ks + WD : steps - 1, e % WD);   // that set was expanded a step ago
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      half8_t bf[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        bf[mt] = *reinterpret_cast<const half8_t*>(&xs[p][(wm * 32 * MT + mt * 32 + ql) * XS + hb * 32 + j * 8]);
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[nt][j], bf[mt], acc[nt][mt], 0, 0, 0);
      expand(j, e + 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(p ^ 1);
    if (SBV && e == SBW - 1) {
      // the next chunk becomes the current one (its loads were issued SBW steps ago)
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt) {
        s8[0][nt] = s8[1][nt];
        b8[0][nt] = b8[1][nt];
      }
      const int c = ks / SBW + 2;
      fetch_sb(c < chunks ? c : chunks - 1, 1);
    }
    __syncthreads();
  };
  if constexpr (SBW == 8) {
    for (int ks = 0; ks < steps; ks += 8) {
      body(ks, StepIndex<0>{});
      body(ks + 1, StepIndex<1>{});
      body(ks + 2, StepIndex<2>{});
      body(ks + 3, StepIndex<3>{});
      body(ks + 4, StepIndex<4>{});
      body(ks + 5, StepIndex<5>{});
      body(ks + 6, StepIndex<6>{});
      body(ks + 7, StepIndex<7>{});
    }
  } else if constexpr (SBW == 4) {
    for (int ks = 0; ks < steps; ks += 4) {
      body(ks, StepIndex<0>{});
      body(ks + 1, StepIndex<1>{});
      body(ks + 2, StepIndex<2>{});
      body(ks + 3, StepIndex<3>{});
    }
  } else if constexpr (SBW == 2) {
    for (int ks = 0; ks < steps; ks += 2) {
      body(ks, StepIndex<0>{});
      body(ks + 1, StepIndex<1>{});
    }
  } else {
    int ks = 0;
    for (; ks + 1 < steps; ks += 2) {
      body(ks, StepIndex<0>{});
      body(ks + 1, StepIndex<1>{});
    }
    if (ks < steps) body(ks, StepIndex<0>{});
  }

  // Accumulator register i of a lane: weight row (output column) 8*(i/4) + 4*hb + i%4 of the
  // tile, x row (output row) ql: four columns (8 bytes) of a row per lane and store, so stores
  // straight from the registers touch 32 output lines 16 bytes at a time, eight times over.  The
  // wave's tile goes through LDS instead (its own region, over the x buffers, which every wave
  // has finished reading) and leaves as whole rows: 16 bytes per lane, a row of the tile per
  // 4 * NTW lanes.
  __syncthreads();
  if (KGRP > 1) {
    // the second group's accumulators through LDS (over the x buffers), lane-contiguous
    float4_t* red = reinterpret_cast<float4_t*>(xs_all) + (wave * (NTW * MT * 4)) * 64 + lane;
    if (grp == 1) {
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4)
            red[((nt * MT + mt) * 4 + i4) * 64] = float4_t{acc[nt][mt][4 * i4], acc[nt][mt][4 * i4 + 1],
                                                           acc[nt][mt][4 * i4 + 2], acc[nt][mt][4 * i4 + 3]};
    }
    __syncthreads();
    if (grp == 0) {
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const float4_t v = red[((nt * MT + mt) * 4 + i4) * 64];
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[nt][mt][4 * i4 + e] += v[e];
          }
    }
    __syncthreads();                                     // the sums are in registers: LDS is free again
    if (grp != 0) return;
  }
  if (SWI) {
    // 16 output columns per 32-row tile: accumulator registers 0..7 are gate rows 8 (i / 4) + 4 hb +
    // i % 4, registers 8..15 the up rows 16 further on
    constexpr int ROWB = 32 * NTW + 16;
    unsigned char* stage = reinterpret_cast<unsigned char*>(xs_all) + wave * (32 * MT * ROWB);
    const int NO = N >> 1;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int i4 = 0; i4 < 2; ++i4) {
          const int n = n0 + nt * 32 + 8 * i4 + 4 * hb;            // gate row; the up row is n + 16
          half4_t o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            half_t g = (half_t)acc[nt][mt][4 * i4 + e], u = (half_t)acc[nt][mt][8 + 4 * i4 + e];
            if (bias && n + 16 < N) {
              g = g + bias[n + e];
              u = u + bias[n + 16 + e];
            }
            const float gf = (float)g;
            const half_t a = (half_t)(gf / (1.0f + expf(-gf)));
            o[e] = (half_t)((float)a * (float)u);
          }
          *reinterpret_cast<half4_t*>(stage + (mt * 32 + ql) * ROWB + nt * 32 + i4 * 16 + hb * 8) = o;
        }
    __builtin_amdgcn_wave_barrier();
    constexpr int LPR = 2 * NTW;                         // lanes per row (16 bytes each)
    constexpr int RPI = 64 / LPR;
    const int pr = lane / LPR, pc = lane % LPR;
#pragma unroll
    for (int r0 = 0; r0 < 32 * MT; r0 += RPI) {
      const int row = r0 + pr;
      const int m = m0 + wm * 32 * MT + row;
      const int n = (n0 >> 1) + pc * 8;
      const half8_t v = *reinterpret_cast<const half8_t*>(stage + row * ROWB + pc * 16);
      if (m < M && n < NO) *reinterpret_cast<half8_t*>(out + (long)m * NO + n) = v;
    }
  } else {
    constexpr int ROWB = 64 * NTW + 16;                  // bytes per staged row (padded)
    unsigned char* stage = reinterpret_cast<unsigned char*>(xs_all) + wave * (32 * MT * ROWB);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          half4_t v = half4_t{(half_t)acc[nt][mt][4 * i4 + 0], (half_t)acc[nt][mt][4 * i4 + 1],
                              (half_t)acc[nt][mt][4 * i4 + 2], (half_t)acc[nt][mt][4 * i4 + 3]};
          const int n = n0 + nt * 32 + 8 * i4 + 4 * hb;
          if (bias && n < N) v += *reinterpret_cast<const half4_t*>(bias + n);
          *reinterpret_cast<half4_t*>(stage + (mt * 32 + ql) * ROWB + nt * 64 + i4 * 16 + hb * 8) = v;
        }
    __builtin_amdgcn_wave_barrier();
    constexpr int LPR = 4 * NTW;                         // lanes per row (16 bytes each)
    constexpr int RPI = 64 / LPR;                        // rows per store instruction
    const int pr = lane / LPR, pc = lane % LPR;
#pragma unroll
    for (int r0 = 0; r0 < 32 * MT; r0 += RPI) {
      const int row = r0 + pr;
      const int m = m0 + wm * 32 * MT + row;
      const int n = n0 + pc * 8;
      const half8_t v = *reinterpret_cast<const half8_t*>(stage + row * ROWB + pc * 16);
      if (m < M && n < N) *reinterpret_cast<half8_t*>(out + (long)m * N + n) = v;
    }
  }
}

template <int NTW, int MT, int SBW, int KGRP = 1, bool SWI = false>
int launch_gemm(const half_t* x, const uint32_t* w, const half_t* s, const half_t* b, const half_t* bias,
                half_t* out, int M, int N, int K, hipStream_t st) {
  constexpr int BMT = 32 * MT;
  constexpr int BN = 128 * NTW;
  static_assert(256 % BMT == 0 && BMT >= 32, "block load mapping");
  const size_t lds_x = KGRP * 2 * (size_t)BMT * XS * sizeof(half_t);
  const size_t lds_out = 4 * (size_t)BMT * (64 * NTW + 16);         // the output tiles of the four waves
  const size_t lds_red = KGRP > 1 ? 4 * (size_t)NTW * MT * 4 * 64 * sizeof(float4_t) : 0;
  size_t lds = lds_x > lds_out ? lds_x : lds_out;
  lds = lds > lds_red ? lds : lds_red;
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_gemm_w4g64_kernel<NTW, MT, SBW, KGRP, SWI>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  const dim3 grid((N + BN - 1) / BN, (M + BMT - 1) / BMT);
  hipLaunchKernelGGL((qmm_gemm_w4g64_kernel<NTW, MT, SBW, KGRP, SWI>), grid, dim3(256 * KGRP), lds, st, x, w, s, b,
                     bias, out, M, N, K);
  return eagle_launch_status();
}


// ------------------------------------------------------------------------------------------
// Up to 32 rows: K slabs, x through LDS a chunk of eight steps at a time, fp32 partial sums as
// the result
// ------------------------------------------------------------------------------------------
// A workgroup of four waves owns 128 weight rows (one 32-row tile per wave) and one K slab of
// `spz` steps (a multiple of eight).  x travels through LDS in chunks of eight steps
// [32 x 512], in the operand order of the weights as above, double buffered: the chunk after
// next is in flight in registers while the waves work on the current one, and the one barrier
// per chunk is all that ties the waves together.  Each lane keeps eight weight loads in flight
// (the register of a step is loaded again for the step eight ahead as soon as it has been
// expanded); scales and biases come eight groups per fetch; four matrix instructions per step.
// Two to four workgroups share a compute unit (33 KB of LDS per x buffer), so one workgroup's
// expansion overlaps another's loads.
// The kernel ends with the fp32 partial tile of its slab, partial[slab][row][column]: adding
// the slabs is left to the kernel that reads the result (normalisation, rotary embedding, or
// slab_sum_kernel below).  A last-arriver reduction inside this kernel (partial store, wait,
// counter, loads of all slabs, store) is a chain of device-scope round trips that took longer
// than the product itself: 14.1 us against 5.7 us for 32 x 4608 x 3584.
constexpr int SLAB_RING = 8;
constexpr int SLAB_ROWS = 32;               // rows of x per accumulator tile
constexpr int SLAB_XR = SLAB_RING * 64 + 8; // LDS row stride of an x chunk in halves
constexpr int SLAB_XBUF = SLAB_ROWS * SLAB_XR;

// RAGGED: K is a multiple of 128 but not of 512.  A slab may then hold any number of steps:
// the last chunk is partial (its loads are repeated from the slab's last step, its extra
// steps are skipped) and scales / biases come two groups per fetch.
// MR: 32-row tiles of x (1: up to 32 rows, 2: 33..64 rows of a tree above 32 tokens).  With two,
// every expanded weight operand feeds two matrix instructions, the x chunk in LDS has 64 rows
// (66 KB per buffer) and the partial tile is [64][N].
// SWI: one slab over all of K (gridDim.y == 1), the weight rows gate and up interleaved in 16-row
// tiles (a wave's 32 rows are one gate tile and its up tile), and the result silu(g) * u as fp16
// [M, N / 2] in `swi_out` (bias [N], interleaved like the rows, or null) instead of partial sums.
// NWV: waves (32-row weight tiles) per workgroup, 4 unless SWI: there the host picks the count
// that fits the launch into one workgroup per compute unit where it can (37888 rows: 296
// workgroups of four waves would leave 40 compute units with two of them and everyone waiting
// for those; 237 of five waves run side by side).  Waves beyond the fourth only multiply.
// WR: register sets of eight weight loads per lane (1: the loads of the next chunk are in flight
// while a chunk is used; 2: those of the next two, for slabs of many chunks, where the time per
// step is the load latency divided by the loads in flight).
// TL: the weights come in the tiled layout (eagle_qmm_tile_w4g64): w is [N/32 tiles][K/64 steps]
// [64 lanes][4 words], one contiguous 1 KB block per wave and step in the order the lanes hold it,
// and s is [N/32 tiles][K/512 chunks][64 lanes][8 halves] with the scales of the chunk's eight
// groups in lanes 0..31 (one row each) and the biases in lanes 32..63; b is not read.  A load
// instruction then touches eight whole cache lines instead of pieces of 32 or 64.
// SUBN: expansion through fp16 subnormals (dequant_word_sub), for |scale| < 0.0624.
template <bool RAGGED, int MR = 1, bool SWI = false, int NWV = 4, int WR = 1, bool TL = false, bool SUBN = false>
__global__ __launch_bounds__(64 * NWV) void qmm_slab_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w, const half_t* __restrict__ s,
    const half_t* __restrict__ b, float* __restrict__ partial, int M, int N, int K, int spz, int xbufs,
    const half_t* __restrict__ swi_bias = nullptr, half_t* __restrict__ swi_out = nullptr) {
  static_assert(SWI || NWV == 4, "the partial-sum epilogue is laid out for four waves");
  static_assert(!TL || !RAGGED, "the tiled layout holds whole chunks");
  extern __shared__ __attribute__((aligned(16))) half_t xlds[];   // one or two x chunks
  constexpr int XBUF = MR * SLAB_XBUF;
  const int tid = threadIdx.x;
  const bool mover = NWV == 4 || tid < 256;  // the threads that carry x into LDS
  const int wave = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int z = blockIdx.y;
  const int G = K >> 6;                      // groups (K steps) per weight row
  const int KW = K >> 3;                     // packed words per weight row
  const int g0 = z * spz;
  const int steps = G - g0 < spz ? G - g0 : spz;   // a multiple of eight unless RAGGED (then even)
  const int chunks = (steps + 7) >> 3;
  const int rem = steps - (chunks - 1) * 8;  // steps of the last chunk
  auto step_of = [&](int i) { return RAGGED && i > steps - 1 ? steps - 1 : i; };

  // thread (xr, xc) moves the 16 bytes at column 64 i + 8 xc of rows xr (and xr + 32) for the
  // steps i of a chunk
  const int xr = tid >> 3, xc = tid & 7;
  const half_t* xp[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    const int row = xr + 32 * r;
    xp[r] = x + (long)(row < M ? row : M - 1) * K + g0 * 64 + xc * 8;
  }
  int nrow = blockIdx.x * (32 * NWV) + wave * 32 + ql;
  if (nrow > N - 1) nrow = N - 1;
  int tile = blockIdx.x * NWV + wave;        // TL: the wave's 32-row tile (rows past N are never stored)
  if (tile > (N >> 5) - 1) tile = (N >> 5) - 1;
  const uint32_t* wp = TL ? w + ((long)tile * G + g0) * 256 + lane * 4 : w + (long)nrow * KW + g0 * 8 + hb * 4;
  const half_t* sp = TL ? s + ((long)tile * (G >> 3) + (g0 >> 3)) * 512 + lane * 8 : s + (long)nrow * G + g0;
  const half_t* bp = TL ? nullptr : b + (long)nrow * G + g0;

  half8_t xreg[MR][SLAB_RING];
  uint4_t wreg[WR][SLAB_RING];
  half8_t s8, b8, s8n, b8n;
  // the packed words of one step of this lane's row (steps past the slab repeat its last one)
  auto wload = [&](int step) {
    return *reinterpret_cast<const uint4_t*>(wp + (step < steps ? step : steps - 1) * (TL ? 256 : 8));
  };
  auto fetch_x = [&](int c) {
    if (!mover) return;
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
      for (int i = 0; i < SLAB_RING; ++i)
        xreg[r][i] = *reinterpret_cast<const half8_t*>(xp[r] + step_of(c * 8 + i) * 64);
  };
  // scales and biases of chunk c: one 16-byte fetch, or four 4-byte fetches kept inside the slab
  auto fetch_sb = [&](int c, half8_t& s_out, half8_t& b_out) {
    if constexpr (TL) {
      // one 16-byte load per lane: scales in the lower half of the wave, biases in the upper
      s_out = *reinterpret_cast<const half8_t*>(sp + c * 512);
    } else if (!RAGGED) {
      s_out = *reinterpret_cast<const half8_t*>(sp + c * 8);
      b_out = *reinterpret_cast<const half8_t*>(bp + c * 8);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int g = c * 8 + 2 * i < steps - 2 ? c * 8 + 2 * i : steps - 2;
        const half2_t sv = *reinterpret_cast<const half2_t*>(sp + g);
        const half2_t bv = *reinterpret_cast<const half2_t*>(bp + g);
        s_out[2 * i] = sv[0];
        s_out[2 * i + 1] = sv[1];
        b_out[2 * i] = bv[0];
        b_out[2 * i + 1] = bv[1];
      }
    }
  };
  auto stash_x = [&](int buf) {
    if (!mover) return;
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
      for (int i = 0; i < SLAB_RING; ++i)
        *reinterpret_cast<half8_t*>(&xlds[buf * XBUF + (xr + 32 * r) * SLAB_XR + i * 64 + xc * 8]) =
            permute8(xreg[r][i]);
  };
  fetch_x(0);
  fetch_sb(0, s8, b8);
#pragma unroll
  for (int i = 0; i < SLAB_RING; ++i) wreg[0][i] = wload(i);
  if constexpr (WR == 2) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < SLAB_RING; ++i) wreg[1][i] = wload(SLAB_RING + i);
  }
  __builtin_amdgcn_sched_barrier(0);
  stash_x(0);
  if (chunks > 1) fetch_x(1);
  __syncthreads();

  float16_t acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[r][i] = 0.f;
  const half_t* xrow = xlds + ql * SLAB_XR + hb * 32;

  // one chunk of eight steps on the x chunk in buffer `buf`; RELOAD: the weight registers are
  // loaded again for the next chunk
  auto chunk = [&](int c, int buf, auto RELOAD, auto PAR) {
    constexpr bool reload = decltype(RELOAD)::value != 0;
    constexpr int par = WR == 2 ? decltype(PAR)::value : 0;   // the register set of this chunk
    if constexpr (TL) {
      // s8 holds what this lane loaded (scales in lanes 0..31, biases in 32..63): exchange the
      // halves of the wave so that every lane has both
      union { half8_t h; uint32_t u[4]; } own, oth;
      own.h = s8;
#pragma unroll
      for (int i = 0; i < 4; ++i) oth.u[i] = __shfl_xor(own.u[i], 32, 64);
      s8 = hb ? oth.h : own.h;
      b8 = hb ? own.h : oth.h;
    }
    if (reload) fetch_sb(c + 1, s8n, b8n);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (RAGGED && !reload && e >= rem) break;            // the last chunk may be partial
      const half_t sc = s8[e], bi = b8[e];
      half8_t af[4];
      if constexpr (SUBN) {
        const half_t s20 = (half_t)((float)sc * 1048576.f);
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = dequant_word_sub(wreg[par][e][j], half2_t{s20, s20}, half2_t{bi, bi});
      } else {
        const half_t bc = (half_t)((float)bi + 8.f * (float)sc);
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = dequant_word_centred(wreg[par][e][j], half2_t{sc, sc}, half2_t{bc, bc});
      }
      if constexpr (WR == 2) wreg[par][e] = wload((c + 2) * 8 + e);
      else if (reload) wreg[0][e] = wload((c + 1) * 8 + e);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const half8_t bf =
              *reinterpret_cast<const half8_t*>(xrow + buf * XBUF + r * SLAB_XBUF + e * 64 + j * 8);
          acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[j], bf, acc[r], 0, 0, 0);
        }
      // (with two chunk bodies per loop iteration the scheduler otherwise hoists the x operand
      // reads of many steps to the top and runs out of registers)
      if constexpr (WR == 2) __builtin_amdgcn_sched_barrier(0);
    }
    if (reload) {
      s8 = s8n;
      b8 = b8n;
    }
  };
  // xbufs == 2: the chunks alternate between two LDS buffers.  xbufs == 1 (a slab of one chunk,
  // or a workgroup that leaves LDS room for a second one on its compute unit): one buffer, and
  // a barrier before it is overwritten.
  const int bmask = xbufs - 1;
  // x of chunk c + 1 (requested before chunk c's weight reloads, so that waiting for it leaves
  // those in flight) into the buffer that chunk c - 1 used: every wave left that one before the
  // barrier that ended chunk c - 1
  auto next_x = [&](int c) {
    if constexpr (WR == 2) __builtin_amdgcn_sched_barrier(0);
    if (xbufs == 1) __syncthreads();
    stash_x((c + 1) & bmask);
    if constexpr (WR == 2) __builtin_amdgcn_sched_barrier(0);
    if (c + 2 < chunks) fetch_x(c + 2);
    __syncthreads();
    if constexpr (WR == 2) __builtin_amdgcn_sched_barrier(0);
  };
  if constexpr (WR == 2) {
    // chunks in pairs (even ones on register set 0, odd ones on set 1), then the last one or two
    int c = 0;
    for (; c + 2 < chunks; c += 2) {
      chunk(c, c & bmask, StepIndex<1>{}, StepIndex<0>{});
      next_x(c);
      chunk(c + 1, (c + 1) & bmask, StepIndex<1>{}, StepIndex<1>{});
      next_x(c + 1);
    }
    if (c + 1 < chunks) {
      chunk(c, c & bmask, StepIndex<1>{}, StepIndex<0>{});
      next_x(c);
      chunk(c + 1, (c + 1) & bmask, StepIndex<0>{}, StepIndex<1>{});
    } else {
      chunk(c, c & bmask, StepIndex<0>{}, StepIndex<0>{});
    }
  } else {
    for (int c = 0; c + 1 < chunks; ++c) {
      chunk(c, c & bmask, StepIndex<1>{}, StepIndex<0>{});
      next_x(c);
    }
    chunk(chunks - 1, (chunks - 1) & bmask, StepIndex<0>{}, StepIndex<0>{});
  }

  // accumulator register i of a lane: weight row 8*(i/4) + 4*hb + i%4 of the wave's tile, x
  // row ql (+ 32 for the second tile).  Through LDS, so that the lanes of a wave store whole
  // 512-byte row segments.
  if (SWI) {
    // registers 0..7 of a lane are gate rows 8 (i / 4) + 4 hb + i % 4 of the wave's tile pair,
    // registers 8..15 the up rows 16 further on: 16 output columns per wave, 64 per workgroup
    constexpr int HS = 16 * NWV + 8;         // halves per row of the output tile in LDS
    half_t* ht = xlds;
    __syncthreads();                         // every wave is done with the x chunks
    const int ng = blockIdx.x * (32 * NWV) + wave * 32;
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
      for (int i4 = 0; i4 < 2; ++i4) {
        const int n = ng + 8 * i4 + 4 * hb;  // gate row; the up row is n + 16
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          half_t g = (half_t)acc[r][4 * i4 + e], u = (half_t)acc[r][8 + 4 * i4 + e];
          if (swi_bias && n + 16 + e < N) {
            g = g + swi_bias[n + e];
            u = u + swi_bias[n + 16 + e];
          }
          const float gf = (float)g;
          const half_t a = (half_t)(gf / (1.0f + expf(-gf)));
          o[e] = (half_t)((float)a * (float)u);
        }
        *reinterpret_cast<half4_t*>(&ht[(ql + 32 * r) * HS + wave * 16 + 8 * i4 + 4 * hb]) = o;
      }
    __syncthreads();
    const int NO = N >> 1;
    constexpr int U = 2 * NWV;               // 16-byte pieces of a row of the tile
    for (int idx = tid; idx < MR * 32 * U; idx += 64 * NWV) {
      const int m = idx / U, c8 = (idx % U) * 8;
      const int no = blockIdx.x * (16 * NWV) + c8;
      if (m < M && no < NO)
        *reinterpret_cast<half8_t*>(swi_out + (size_t)m * NO + no) = *reinterpret_cast<const half8_t*>(&ht[m * HS + c8]);
    }
    return;
  }
  constexpr int OS = 128 + 4;                // floats per row of the tile in LDS
  float* ot = reinterpret_cast<float*>(xlds);
  __syncthreads();                           // every wave is done with the x chunks
#pragma unroll
  for (int r = 0; r < MR; ++r)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4)
      *reinterpret_cast<float4_t*>(&ot[(ql + 32 * r) * OS + wave * 32 + 8 * i4 + 4 * hb]) =
          float4_t{acc[r][4 * i4], acc[r][4 * i4 + 1], acc[r][4 * i4 + 2], acc[r][4 * i4 + 3]};
  __syncthreads();
  float* dst = partial + (size_t)z * (MR * SLAB_ROWS) * N;
  const int c = (tid & 31) * 4;
  const int n = blockIdx.x * 128 + c;
#pragma unroll
  for (int pass = 0; pass < 4 * MR; ++pass) {
    const int m = pass * 8 + (tid >> 5);
    if (m < M && n < N)
      *reinterpret_cast<float4_t*>(dst + (size_t)m * N + n) = *reinterpret_cast<const float4_t*>(&ot[m * OS + c]);
  }
}

// ------------------------------------------------------------------------------------------
// The same two products (partial sums of a K slab; gate|up with the SwiGLU epilogue) with two
// waves per weight tile and waves of their own for x
// ------------------------------------------------------------------------------------------
// What bounds the kernel above at 32 rows is the rate at which a compute unit takes in bytes
// (its weight tiles and the x chunks it re-reads from L2 alike) and the time a wave spends per
// tile and K step when it has a SIMD to itself.  Here a workgroup owns TILES 32-row weight tiles
// and one K slab of whole chunks (tiled weight layout only), and
//   * two streaming waves share a weight tile: each takes four of a chunk's eight steps (a
//     whole 128-byte line of every weight row of the tile per chunk) and keeps the loads of
//     BURST_CA chunks in flight, issued in the order they are needed, scales and biases first:
//     loads retire in issue order, and every request of a long slab issued at the start puts
//     the first chunk, which the waves wait for, behind microseconds of later ones.
//     The chunk loop is unrolled over a compile-time chunk count, all loads unconditional;
//   * BURST_MOVERS more waves only carry x: a whole chunk per step of their loop (global ->
//     registers -> LDS in operand order, two chunks in flight in registers, BURST_XB buffers in
//     LDS), so that the streaming waves' in-order load counters never wait for an x load;
//   * one LDS-only barrier per chunk; at the end the second wave of a tile hands its
//     accumulators to the first through LDS, which runs the epilogue of the kernel above.
// SUBN: expansion through fp16 subnormals (dequant_word_sub), for |scale| < 0.0624.
constexpr int BURST_CA = 2;                  // chunks of weight loads in flight per wave
constexpr int BURST_MOVERS = 4;              // waves that only carry x
constexpr int BURST_XB = 3;                  // x chunks in LDS
constexpr int BURST_SPW = 4;                 // steps of a chunk per streaming wave

template <bool SUBN, int NCH>
__device__ inline void burst_stream(const uint32_t* __restrict__ wp, const half_t* __restrict__ sp, int kp, int hb,
                                    const half_t* xrow, float16_t& acc) {
  // wp: the wave's first block of the tiled weights (+ lane), 256 words per step; sp: the
  // tile's first block of scales | biases (+ lane), 512 halves per chunk
  uint4_t wreg[BURST_CA][BURST_SPW];
  half8_t sb[BURST_CA];
  constexpr int PRE = NCH < BURST_CA ? NCH : BURST_CA;
  // scales and biases first, then the weights chunk by chunk: loads retire in issue order, and
  // the first chunk must not wait behind the requests of the later ones
#pragma unroll
  for (int c = 0; c < PRE; ++c) sb[c] = *reinterpret_cast<const half8_t*>(sp + c * 512);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int c = 0; c < PRE; ++c) {
#pragma unroll
    for (int e = 0; e < BURST_SPW; ++e) wreg[c][e] = *reinterpret_cast<const uint4_t*>(wp + (c * 8 + e) * 256);
    __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();                           // x chunk 0 is in LDS
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    constexpr int XBUF = SLAB_XBUF;
    const int slot = c % BURST_CA;
    // this lane loaded eight scales (lanes 0..31) or biases (32..63); the wave's four steps are
    // words 2 kp, 2 kp + 1; exchange the halves of the wave so that every lane has both
    union { half8_t h; uint32_t u[4]; } own;
    own.h = sb[slot];
    const uint32_t m0 = kp ? own.u[2] : own.u[0], m1 = kp ? own.u[3] : own.u[1];
    const uint32_t o0 = __shfl_xor(m0, 32, 64), o1 = __shfl_xor(m1, 32, 64);
    union { uint32_t u[2]; half4_t h; } sc4, bi4;
    sc4.u[0] = hb ? o0 : m0;
    sc4.u[1] = hb ? o1 : m1;
    bi4.u[0] = hb ? m0 : o0;
    bi4.u[1] = hb ? m1 : o1;
    if (c + BURST_CA < NCH) {
      sb[slot] = *reinterpret_cast<const half8_t*>(sp + (c + BURST_CA) * 512);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int e = 0; e < BURST_SPW; ++e) {
      const half_t sc = sc4.h[e], bi = bi4.h[e];
      half8_t af[4];
      if constexpr (SUBN) {
        const half_t s20 = (half_t)((float)sc * 1048576.f);
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = dequant_word_sub(wreg[slot][e][j], half2_t{s20, s20}, half2_t{bi, bi});
      } else {
        const half_t bc = (half_t)((float)bi + 8.f * (float)sc);
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = dequant_word_centred(wreg[slot][e][j], half2_t{sc, sc}, half2_t{bc, bc});
      }
      if (c + BURST_CA < NCH)
        wreg[slot][e] = *reinterpret_cast<const uint4_t*>(wp + ((c + BURST_CA) * 8 + e) * 256);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half8_t bf = *reinterpret_cast<const half8_t*>(xrow + (c % BURST_XB) * XBUF + e * 64 + j * 8);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[j], bf, acc, 0, 0, 0);
      }
      if (c + BURST_CA < NCH) __builtin_amdgcn_sched_barrier(0);   // keeps the reloads in step order
    }
    __syncthreads();                         // every wave is done with chunk c; chunk c + 1 is in LDS
  }
}

template <int TILES, bool SWI, bool SUBN, int NCH, int NLAST>
__global__ __launch_bounds__(64 * (2 * TILES + BURST_MOVERS)) void qmm_burst_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w, const half_t* __restrict__ s,
    const half_t* __restrict__ b, float* __restrict__ partial, int M, int N, int K, int spz,
    const half_t* __restrict__ swi_bias, half_t* __restrict__ swi_out) {
  extern __shared__ __attribute__((aligned(16))) half_t xlds[];   // three x chunks
  constexpr int NSW = 2 * TILES;             // streaming waves
  constexpr int NT = 64 * (NSW + BURST_MOVERS);
  constexpr int XBUF = SLAB_XBUF;
  const int tid = threadIdx.x;
  const int wv = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int z = blockIdx.y;
  const int G = K >> 6;
  const int g0 = z * spz;
  const int steps = G - g0 < spz ? G - g0 : spz;   // a multiple of eight
  const int chunks = steps >> 3;                    // NCH, or NLAST for the last slab
  const int t = wv % TILES, kp = wv / TILES;        // tile and half of the chunk of a streaming wave
  float16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;

  if (wv >= NSW) {
    // piece 256 i + mt of a chunk: row (256 i + mt) / 64, 16-byte column (256 i + mt) % 64.
    // Two chunks are in flight in registers and up to three sit in LDS: chunk c + 1 is written
    // during chunk c (into the buffer chunk c - 2 used) and was requested two chunks earlier.
    const int mt = tid - 64 * NSW;
    const int r0 = mt >> 6, c8 = mt & 63;
    half8_t xr[2][8];
    const half_t* xp[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 4 * i + r0;
      xp[i] = x + (long)(row < M ? row : M - 1) * K + g0 * 64 + c8 * 8;
    }
    const int last = chunks - 1;
    auto fetch = [&](int c, auto SET) {
      constexpr int set = decltype(SET)::value;
      const int cc = c < last ? c : last;
#pragma unroll
      for (int i = 0; i < 8; ++i) xr[set][i] = *reinterpret_cast<const half8_t*>(xp[i] + cc * 512);
    };
    auto stash = [&](int c, auto SET) {
      constexpr int set = decltype(SET)::value;
      const int buf = c % BURST_XB;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *reinterpret_cast<half8_t*>(&xlds[buf * XBUF + (4 * i + r0) * SLAB_XR + c8 * 8]) = permute8(xr[set][i]);
    };
    fetch(0, StepIndex<0>{});
    fetch(1, StepIndex<1>{});
    stash(0, StepIndex<0>{});
    fetch(2, StepIndex<0>{});
    __syncthreads();
    // during chunk c: chunk c + 1 goes into LDS (requested two chunks ago), chunk c + 3 is requested
    for (int c = 0; c < chunks; c += 2) {
      stash(c + 1, StepIndex<1>{});
      fetch(c + 3, StepIndex<1>{});
      __syncthreads();
      if (c + 1 < chunks) {
        stash(c + 2, StepIndex<0>{});
        fetch(c + 4, StepIndex<0>{});
        __syncthreads();
      }
    }
  } else {
    int tile = blockIdx.x * TILES + t;         // rows past N are never stored
    if (tile > (N >> 5) - 1) tile = (N >> 5) - 1;
    const uint32_t* wp = w + ((long)tile * G + g0 + kp * BURST_SPW) * 256 + lane * 4;
    const half_t* sp = s + ((long)tile * (G >> 3) + (g0 >> 3)) * 512 + lane * 8;
    const half_t* xrow = xlds + ql * SLAB_XR + hb * 32 + kp * BURST_SPW * 64;
    if (NCH == NLAST || chunks == NCH) burst_stream<SUBN, NCH>(wp, sp, kp, hb, xrow, acc);
    else burst_stream<SUBN, NLAST>(wp, sp, kp, hb, xrow, acc);
  }

  // the second wave of a tile hands its accumulators over (register i of lane l at [tile][i][l]),
  // behind the output tile
  constexpr int OUT_BYTES = SWI ? 32 * (16 * TILES + 8) * 2 : 32 * (32 * TILES + 4) * 4;
  float* ex = reinterpret_cast<float*>(reinterpret_cast<char*>(xlds) + ((OUT_BYTES + 255) / 256) * 256) + t * (16 * 64) + lane;
  if (wv < NSW && kp == 1) {
#pragma unroll
    for (int i = 0; i < 16; ++i) ex[i * 64] = acc[i];
  }
  __syncthreads();
  const bool owner = wv < NSW && kp == 0;
  if (owner) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] += ex[i * 64];
  }
  if constexpr (SWI) {
    constexpr int HS = 16 * TILES + 8;       // halves per row of the output tile in LDS
    half_t* ht = xlds;
    if (owner) {
      const int ng = blockIdx.x * (32 * TILES) + t * 32;
#pragma unroll
      for (int i4 = 0; i4 < 2; ++i4) {
        const int n = ng + 8 * i4 + 4 * hb;  // gate row; the up row is n + 16
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          half_t g = (half_t)acc[4 * i4 + e], u = (half_t)acc[8 + 4 * i4 + e];
          if (swi_bias && n + 16 + e < N) {
            g = g + swi_bias[n + e];
            u = u + swi_bias[n + 16 + e];
          }
          const float gf = (float)g;
          const half_t a = (half_t)(gf / (1.0f + expf(-gf)));
          o[e] = (half_t)((float)a * (float)u);
        }
        *reinterpret_cast<half4_t*>(&ht[ql * HS + t * 16 + 8 * i4 + 4 * hb]) = o;
      }
    }
    __syncthreads();
    const int NO = N >> 1;
    constexpr int U = 2 * TILES;             // 16-byte pieces of a row of the tile
    for (int idx = tid; idx < 32 * U; idx += NT) {
      const int m = idx / U, c8 = (idx % U) * 8;
      const int no = blockIdx.x * (16 * TILES) + c8;
      if (m < M && no < NO)
        *reinterpret_cast<half8_t*>(swi_out + (size_t)m * NO + no) = *reinterpret_cast<const half8_t*>(&ht[m * HS + c8]);
    }
  } else {
    constexpr int OS = 32 * TILES + 4;       // floats per row of the tile in LDS
    float* ot = reinterpret_cast<float*>(xlds);
    if (owner) {
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        *reinterpret_cast<float4_t*>(&ot[ql * OS + t * 32 + 8 * i4 + 4 * hb]) =
            float4_t{acc[4 * i4], acc[4 * i4 + 1], acc[4 * i4 + 2], acc[4 * i4 + 3]};
    }
    __syncthreads();
    float* dst = partial + (size_t)z * SLAB_ROWS * N;
    constexpr int U = 8 * TILES;             // 16-byte pieces of a row of the tile
    for (int idx = tid; idx < 32 * U; idx += NT) {
      const int m = idx / U, c4 = (idx % U) * 4;
      const int n = blockIdx.x * (32 * TILES) + c4;
      if (m < M && n < N)
        *reinterpret_cast<float4_t*>(dst + (size_t)m * N + n) = *reinterpret_cast<const float4_t*>(&ot[m * OS + c4]);
    }
  }
}

template <int TILES, bool SWI, bool SUBN, int NCH, int NLAST>
int launch_burst(const half_t* x, const uint32_t* w, const half_t* s, const half_t* b, float* partial, int M,
                 int N, int K, int spz, int slabs, const half_t* bias, half_t* out, hipStream_t st) {
  const size_t lds = BURST_XB * (size_t)SLAB_XBUF * sizeof(half_t);
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_burst_w4g64_kernel<TILES, SWI, SUBN, NCH, NLAST>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  const dim3 grid((N + 32 * TILES - 1) / (32 * TILES), slabs);
  hipLaunchKernelGGL((qmm_burst_w4g64_kernel<TILES, SWI, SUBN, NCH, NLAST>), grid,
                     dim3(64 * (2 * TILES + BURST_MOVERS)), lds, st, x, w, s, b, partial, M, N, K, spz, bias, out);
  return eagle_launch_status();
}

// ------------------------------------------------------------------------------------------
// The whole product of up to 32 rows with a matrix of very many rows (a vocabulary projection),
// fp16 out, from the tiled weight layout
// ------------------------------------------------------------------------------------------
// A compute unit takes in bytes at a fixed rate, the x chunks it re-reads from L2 included, so
// the cheapest division gives every compute unit ONE pass over x: a workgroup per compute unit
// owns 2 NSW 32-row weight tiles over all of K.  Each of its NSW streaming waves owns two tiles
// and walks K once: per chunk of eight steps sixteen (step, tile) items, the x operand of a step
// read from LDS once for both tiles, the packed weights of the next eight items in flight in a
// register ring (the register of an item is loaded again for the item eight ahead as soon as it
// has been expanded; all loads unconditional, the chunk loop's body the same every time, so the
// wait counts are exact).  Two more waves only carry x (as in the kernel above).  At the end the
// tile [32 x 64 NSW] goes through LDS and is stored as whole rows, bias added in fp16.
constexpr int ROWS_MOVERS = 2;

template <int NSW, bool SUBN>
__global__ __launch_bounds__(64 * (NSW + ROWS_MOVERS)) void qmm_rows_tiled_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w, const half_t* __restrict__ s,
    const half_t* __restrict__ bias, half_t* __restrict__ out, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(16))) half_t xlds[];   // three x chunks, then the output tile
  constexpr int NT = 64 * (NSW + ROWS_MOVERS);
  constexpr int XBUF = SLAB_XBUF;
  // (step, tile) items of packed weights in flight per lane.  Sixteen (a whole chunk) were slower
  // (74 against 68 us for 32 x 152064 x 3584) and four the same: the depth is not what bounds it.
  constexpr int ROWS_RING = 8;
  const int tid = threadIdx.x;
  const int wv = tid >> 6, lane = tid & 63;
  const int ql = lane & 31, hb = lane >> 5;
  const int G = K >> 6;
  const int chunks = G >> 3;
  float16_t acc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;

  if (wv >= NSW) {
    // piece 128 i + mt of a chunk: row (128 i + mt) / 64, 16-byte column (128 i + mt) % 64
    const int mt = tid - 64 * NSW;
    const int r0 = mt >> 6, c8 = mt & 63;
    half8_t xr[2][16];
    const half_t* xb = x + c8 * 8;
    uint32_t xo[16];                                 // element offsets of the thread's rows (M * K < 2^31)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 2 * i + r0;
      xo[i] = (uint32_t)(row < M ? row : M - 1) * (uint32_t)K;
    }
    const int last = chunks - 1;
    auto fetch = [&](int c, auto SET) {
      constexpr int set = decltype(SET)::value;
      const int cc = c < last ? c : last;
#pragma unroll
      for (int i = 0; i < 16; ++i) xr[set][i] = *reinterpret_cast<const half8_t*>(xb + (xo[i] + (uint32_t)(cc * 512)));
    };
    auto stash = [&](int c, auto SET) {
      constexpr int set = decltype(SET)::value;
      const int buf = c % BURST_XB;
#pragma unroll
      for (int i = 0; i < 16; ++i)
        *reinterpret_cast<half8_t*>(&xlds[buf * XBUF + (2 * i + r0) * SLAB_XR + c8 * 8]) = permute8(xr[set][i]);
    };
    fetch(0, StepIndex<0>{});
    fetch(1, StepIndex<1>{});
    stash(0, StepIndex<0>{});
    fetch(2, StepIndex<0>{});
    __syncthreads();
    for (int c = 0; c < chunks; c += 2) {
      stash(c + 1, StepIndex<1>{});
      fetch(c + 3, StepIndex<1>{});
      __syncthreads();
      if (c + 1 < chunks) {
        stash(c + 2, StepIndex<0>{});
        fetch(c + 4, StepIndex<0>{});
        __syncthreads();
      }
    }
  } else {
    const int ntiles = N >> 5;
    const uint32_t* wp[2];
    const half_t* sp[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      int tile = (blockIdx.x * NSW + wv) * 2 + j;    // rows past N are never stored
      if (tile > ntiles - 1) tile = ntiles - 1;
      wp[j] = w + (long)tile * G * 256 + lane * 4;
      sp[j] = s + (long)tile * (G >> 3) * 512 + lane * 8;
    }
    const half_t* xrow = xlds + ql * SLAB_XR + hb * 32;
    uint4_t wreg[ROWS_RING];                         // item i = 2 e + j (step e of the chunk, tile j) in register i % ROWS_RING
    half8_t sb[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) sb[j] = *reinterpret_cast<const half8_t*>(sp[j]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < ROWS_RING; ++i) wreg[i] = *reinterpret_cast<const uint4_t*>(wp[i & 1] + (i >> 1) * 256);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();                                 // x chunk 0 is in LDS
    const int last = chunks - 1;
    for (int c = 0; c < chunks; ++c) {
      // this lane loaded eight scales (lanes 0..31) or biases (32..63) per tile; exchange the
      // halves of the wave so that every lane has both, then request the next chunk's
      const int cn = c < last ? c + 1 : last;
      union { half8_t h; uint32_t u[4]; } own, oth;
      half8_t s8[2], b8[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        own.h = sb[j];
#pragma unroll
        for (int i = 0; i < 4; ++i) oth.u[i] = __shfl_xor(own.u[i], 32, 64);
        s8[j] = hb ? oth.h : own.h;
        b8[j] = hb ? own.h : oth.h;
        sb[j] = *reinterpret_cast<const half8_t*>(sp[j] + cn * 512);
      }
      __builtin_amdgcn_sched_barrier(0);
      const half_t* xc = xrow + (c % BURST_XB) * XBUF;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        half8_t bf[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) bf[k] = *reinterpret_cast<const half8_t*>(xc + e * 64 + k * 8);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int r = (2 * e + j) % ROWS_RING;
          const half_t sc = s8[j][e], bi = b8[j][e];
          half8_t af[4];
          if constexpr (SUBN) {
            const half_t s20 = (half_t)((float)sc * 1048576.f);
#pragma unroll
            for (int k = 0; k < 4; ++k) af[k] = dequant_word_sub(wreg[r][k], half2_t{s20, s20}, half2_t{bi, bi});
          } else {
            const half_t bc = (half_t)((float)bi + 8.f * (float)sc);
#pragma unroll
            for (int k = 0; k < 4; ++k) af[k] = dequant_word_centred(wreg[r][k], half2_t{sc, sc}, half2_t{bc, bc});
          }
          // the item ROWS_RING ahead: a later step of this chunk, or a step of the next
          constexpr int AH = ROWS_RING / 2;          // steps ahead
          wreg[r] = *reinterpret_cast<const uint4_t*>(wp[j] + ((e + AH < 8 ? c * 8 + e + AH : cn * 8 + e + AH - 8)) * 256);
#pragma unroll
          for (int k = 0; k < 4; ++k) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[k], bf[k], acc[j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);           // keeps the reloads in item order
      }
      __syncthreads();                               // every wave is done with chunk c; chunk c + 1 is in LDS
    }
  }

  // accumulator register i of a lane: weight row 8 (i / 4) + 4 hb + i % 4 of the tile, x row ql
  constexpr int HS = 64 * NSW + 8;                   // halves per row of the output tile in LDS
  half_t* ht = xlds;
  if (wv < NSW) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = (2 * wv + j) * 32;
      const int n0 = blockIdx.x * (64 * NSW) + col;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int n = n0 + 8 * i4 + 4 * hb;
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[e] = (half_t)acc[j][4 * i4 + e];
          if (bias && n + e < N) o[e] = o[e] + bias[n + e];
        }
        *reinterpret_cast<half4_t*>(&ht[ql * HS + col + 8 * i4 + 4 * hb]) = o;
      }
    }
  }
  __syncthreads();
  constexpr int U = 8 * NSW;                         // 16-byte pieces of a row of the tile
  for (int idx = tid; idx < 32 * U; idx += NT) {
    const int m = idx / U, c8 = (idx % U) * 8;
    const int n = blockIdx.x * (64 * NSW) + c8;
    if (m < M && n < N)
      *reinterpret_cast<half8_t*>(out + (size_t)m * N + n) = *reinterpret_cast<const half8_t*>(&ht[m * HS + c8]);
  }
}

template <int NSW, bool SUBN>
int launch_rows_tiled(const half_t* x, const uint32_t* w, const half_t* s, const half_t* bias, half_t* out, int M,
                      int N, int K, hipStream_t st) {
  const size_t lds = BURST_XB * (size_t)SLAB_XBUF * sizeof(half_t);
  static_assert(BURST_XB * SLAB_XBUF >= 32 * (64 * NSW + 8), "the output tile reuses the x buffers");
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_rows_tiled_kernel<NSW, SUBN>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  const int blocks = ((N >> 5) + 2 * NSW - 1) / (2 * NSW);
  hipLaunchKernelGGL((qmm_rows_tiled_kernel<NSW, SUBN>), dim3(blocks), dim3(64 * (NSW + ROWS_MOVERS)), lds, st, x, w, s,
                     bias, out, M, N, K);
  return eagle_launch_status();
}

// The tiled layout of a weight matrix (see TL above) from the row-major one: thread = one 16-byte
// piece of the output.
__global__ void tile_weights_kernel(const uint32_t* __restrict__ w, const half_t* __restrict__ s,
                                    const half_t* __restrict__ b, uint32_t* __restrict__ wt,
                                    half_t* __restrict__ sbt, int N, int K) {
  const int G = K >> 6, KW = K >> 3;
  const long nw = (long)(N >> 5) * G * 64;             // pieces of wt
  const long nsb = (long)(N >> 5) * (G >> 3) * 64;     // pieces of sbt
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < nw) {
    const int lane = (int)(idx & 63);
    const long ts = idx >> 6;
    const int step = (int)(ts % G);
    const long tile = ts / G;
    const long row = tile * 32 + (lane & 31);
    *reinterpret_cast<uint4_t*>(wt + idx * 4) =
        *reinterpret_cast<const uint4_t*>(w + row * KW + step * 8 + (lane >> 5) * 4);
  } else if (idx < nw + nsb) {
    const long i = idx - nw;
    const int lane = (int)(i & 63);
    const long tc = i >> 6;
    const int chunk = (int)(tc % (G >> 3));
    const long tile = tc / (G >> 3);
    const long row = tile * 32 + (lane & 31);
    const half_t* src = (lane >> 5) ? b : s;
    *reinterpret_cast<half8_t*>(sbt + i * 8) = *reinterpret_cast<const half8_t*>(src + row * G + chunk * 8);
  }
}

// out[m][n] = fp16(sum over the slabs, in slab order) (+ bias): the plain reader of partial sums
__global__ void slab_sum_kernel(const float* __restrict__ partial, int nslab, const half_t* __restrict__ bias,
                                half_t* __restrict__ out, int M, int N) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_row = N >> 3;
  if (idx >= (long)M * per_row) return;
  const int m = (int)(idx / per_row), n = (int)(idx % per_row) * 8;
  const half8_t v = eagle_slab_sum8(partial, nslab, (size_t)eagle_slab_rows(M) * N, (size_t)m * N + n, bias ? bias + n : nullptr);
  *reinterpret_cast<half8_t*>(out + (size_t)m * N + n) = v;
}

}  // namespace


EAGLE_EXPORT int eagle_qmm_slab_count(int K, int steps_per_slab) {
  if (K < 128 || (K % 128) != 0 || steps_per_slab < 8 || (steps_per_slab % 8) != 0 || steps_per_slab > 4096)
    return 0;
  return (K / 64 + steps_per_slab - 1) / steps_per_slab;
}

EAGLE_EXPORT int eagle_qmm_slab_steps(int M, int N, int K) {
  // Measured at 8, 16 and 32 rows on the projections of the 7B and 8B models, alone and inside
  // the verification step: the slab form wins for the projections with a few thousand weight
  // rows (q|k|v, o, down: 5-8 us against 9-14 us, 14 us against 24 us); the streaming kernel
  // keeps gate|up (its SwiGLU epilogue saves a launch) and the vocabulary projection.  Eight
  // steps per slab while that gives at most eight slabs, otherwise longer slabs so that the
  // reader of the result has about ten slabs to add.
  if (M < 1 || M > 2 * SLAB_ROWS || N < 8 || (N % 8) != 0 || K < 512 || (K % 512) != 0) return 0;
  if (N > 8192) return 0;
  const int G = K / 64;
  return G <= 64 ? 8 : G <= 128 ? 16 : 32;
}

EAGLE_EXPORT size_t eagle_qmm_slab_partial_bytes(int N, int K, int steps_per_slab) {
  if (N < 1) return 0;
  return (size_t)eagle_qmm_slab_count(K, steps_per_slab) * SLAB_ROWS * N * sizeof(float);
}

EAGLE_EXPORT size_t eagle_qmm_slab_partial_bytes_rows(int M, int N, int K, int steps_per_slab) {
  if (N < 1 || M < 1 || M > 2 * SLAB_ROWS) return 0;
  return (size_t)eagle_qmm_slab_count(K, steps_per_slab) * eagle_slab_rows(M) * N * sizeof(float);
}

EAGLE_EXPORT int eagle_qmm_slab_partial_w4g64(const void* x, const uint32_t* wq, const void* scales,
                                              const void* biases, float* partial, size_t partial_bytes,
                                              int M, int N, int K, int group_size, int bits,
                                              int steps_per_slab, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !partial) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (M < 1 || M > 2 * SLAB_ROWS || N < 8 || (N % 8) != 0 || K < 128 || (K % 128) != 0) return EAGLE_ERR_SHAPE;
  const int slabs = eagle_qmm_slab_count(K, steps_per_slab);
  if (slabs < 1 || slabs > 65535) return EAGLE_ERR_SHAPE;
  const bool ragged = (K % 512) != 0;
  const uintptr_t sb_mask = ragged ? 3u : 15u;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(partial) ||
      (reinterpret_cast<uintptr_t>(scales) & sb_mask) || (reinterpret_cast<uintptr_t>(biases) & sb_mask))
    return EAGLE_ERR_ALIGN;
  if (partial_bytes < eagle_qmm_slab_partial_bytes_rows(M, N, K, steps_per_slab)) return EAGLE_ERR_WORKSPACE;
  const int mr = M > SLAB_ROWS ? 2 : 1;
  const int bufs = steps_per_slab > SLAB_RING ? 2 : 1;
  const size_t lds = (size_t)bufs * mr * SLAB_XBUF * sizeof(half_t);
  static bool configured = false;
  if (!configured) {
    const int most = 2 * SLAB_XBUF * (int)sizeof(half_t);
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 1>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<true, 1>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 2>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<true, 2>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((N + 127) / 128, slabs);
#define EAGLE_SLAB_LAUNCH(RAG, MRV)                                                                      \
  hipLaunchKernelGGL((qmm_slab_w4g64_kernel<RAG, MRV>), grid, dim3(256), lds, st,                        \
                     static_cast<const half_t*>(x), wq, static_cast<const half_t*>(scales),              \
                     static_cast<const half_t*>(biases), partial, M, N, K, steps_per_slab, bufs)
  if (ragged) {
    if (mr == 2) EAGLE_SLAB_LAUNCH(true, 2); else EAGLE_SLAB_LAUNCH(true, 1);
  } else {
    if (mr == 2) EAGLE_SLAB_LAUNCH(false, 2); else EAGLE_SLAB_LAUNCH(false, 1);
  }
#undef EAGLE_SLAB_LAUNCH
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmm_slab_swiglu_supported(int M, int N, int K) {
  return M >= 1 && M <= 2 * SLAB_ROWS && N >= 32 && (N % 32) == 0 && K >= 128 && (K % 128) == 0 && K <= 65536;
}

EAGLE_EXPORT int eagle_qmm_slab_swiglu_preferred(int M, int N, int K) {
  // Measured against the streaming kernel's SwiGLU form (gate|up of the 7B and 8B shapes, us):
  //   rows          8     16     24     32     40     64
  //   7B slab    29.6   28.7   28.6   28.8   34.6   35.9      (237 workgroups of five waves)
  //   7B stream  23.5   22.7   27.6   28.7   48.5   56.1      (40, 64: two launches)
  //   8B slab    23.5   24.1   24.8   24.3   30.7   31.3      (224 workgroups of four waves)
  //   8B stream  20.8   21.2   26.1   27.0   45.5   52.8
  // so: always above 32 rows; from 24 rows where workgroups of four waves fill at least half of
  // the compute units and at most all of them.
  if (!eagle_qmm_slab_swiglu_supported(M, N, K)) return 0;
  if (M > SLAB_ROWS) return 1;
  const long blocks = (N + 127) / 128;
  return M >= 24 && blocks > NUM_CU / 2 && blocks <= NUM_CU && K >= 2048;
}

EAGLE_EXPORT int eagle_qmm_slab_swiglu_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                                 const void* biases, const void* bias, void* out, int M,
                                                 int N, int K, int group_size, int bits,
                                                 eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (!eagle_qmm_slab_swiglu_supported(M, N, K)) return EAGLE_ERR_SHAPE;
  const bool ragged = (K % 512) != 0;
  const uintptr_t sb_mask = ragged ? 3u : 15u;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(out) ||
      (reinterpret_cast<uintptr_t>(scales) & sb_mask) || (reinterpret_cast<uintptr_t>(biases) & sb_mask) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  const int mr = M > SLAB_ROWS ? 2 : 1;
  const int steps = K / 64;                      // one slab over all of K
  // waves per workgroup: the fewest that give every compute unit at most one workgroup
  int nwv = 4;
  while (nwv < 8 && (N + 32 * nwv - 1) / (32 * nwv) > NUM_CU) nwv += (nwv == 6 ? 2 : 1);
  const int blocks = (N + 32 * nwv - 1) / (32 * nwv);
  // two x buffers, except that with 64 rows they would fill the LDS of a compute unit: when the
  // launch puts two workgroups on some compute units anyway, one buffer each, so that the two
  // fill each other's waits
  const int bufs = steps > SLAB_RING && !(mr == 2 && blocks > NUM_CU) ? 2 : 1;
  const size_t lds = (size_t)bufs * mr * SLAB_XBUF * sizeof(half_t);
  static bool configured = false;
  if (!configured) {
    const int most = 2 * SLAB_XBUF * (int)sizeof(half_t);
    bool ok = true;
#define EAGLE_SLAB_SWI_ATTR(NW)                                                                                  \
  ok = ok &&                                                                                                     \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 1, true, NW, 2>),            \
                           hipFuncAttributeMaxDynamicSharedMemorySize, most) == hipSuccess &&                    \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<true, 1, true, NW, 2>),             \
                           hipFuncAttributeMaxDynamicSharedMemorySize, most) == hipSuccess &&                    \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 2, true, NW, 1>),            \
                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) == hipSuccess &&                \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<true, 2, true, NW, 1>),             \
                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) == hipSuccess
    EAGLE_SLAB_SWI_ATTR(4);
    EAGLE_SLAB_SWI_ATTR(5);
    EAGLE_SLAB_SWI_ATTR(6);
    EAGLE_SLAB_SWI_ATTR(8);
#undef EAGLE_SLAB_SWI_ATTR
    if (!ok) return EAGLE_ERR_HIP;
    configured = true;
  }
  const dim3 grid(blocks, 1);
  hipStream_t st = static_cast<hipStream_t>(stream);
#define EAGLE_SLAB_SWI_LAUNCH(RAG, MRV, NW)                                                              \
  hipLaunchKernelGGL((qmm_slab_w4g64_kernel<RAG, MRV, true, NW, (MRV == 1 ? 2 : 1)>), grid, dim3(64 * NW), lds, st, \
                     static_cast<const half_t*>(x), wq, static_cast<const half_t*>(scales),              \
                     static_cast<const half_t*>(biases), (float*)nullptr, M, N, K, steps, bufs,          \
                     static_cast<const half_t*>(bias), static_cast<half_t*>(out))
#define EAGLE_SLAB_SWI_NW(NW)                                                                            \
  if (ragged) {                                                                                          \
    if (mr == 2) EAGLE_SLAB_SWI_LAUNCH(true, 2, NW); else EAGLE_SLAB_SWI_LAUNCH(true, 1, NW);            \
  } else {                                                                                               \
    if (mr == 2) EAGLE_SLAB_SWI_LAUNCH(false, 2, NW); else EAGLE_SLAB_SWI_LAUNCH(false, 1, NW);          \
  }
  switch (nwv) {
    case 4: EAGLE_SLAB_SWI_NW(4) break;
    case 5: EAGLE_SLAB_SWI_NW(5) break;
    case 6: EAGLE_SLAB_SWI_NW(6) break;
    default: EAGLE_SLAB_SWI_NW(8) break;
  }
#undef EAGLE_SLAB_SWI_NW
#undef EAGLE_SLAB_SWI_LAUNCH
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_slab_sum_f16(const float* partial, int slabs, const void* bias, void* out, int M,
                                    int N, eagle_stream_t stream) {
  if (!partial || !out) return EAGLE_ERR_NULL;
  if (slabs < 1 || M < 1 || M > 2 * SLAB_ROWS || N < 8 || (N % 8) != 0) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(partial) || !eagle_aligned16(out) || (bias && !eagle_aligned16(bias))) return EAGLE_ERR_ALIGN;
  const long total = (long)M * (N / 8);
  hipLaunchKernelGGL(slab_sum_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), partial, slabs, static_cast<const half_t*>(bias),
                     static_cast<half_t*>(out), M, N);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmm_tiled_supported(int M, int N, int K) {
  return M >= 1 && M <= 2 * SLAB_ROWS && N >= 32 && (N % 32) == 0 && K >= 512 && (K % 512) == 0 && K <= 65536;
}

EAGLE_EXPORT size_t eagle_qmm_tiled_sb_bytes(int N, int K) {
  if (N < 32 || (N % 32) != 0 || K < 512 || (K % 512) != 0) return 0;
  return (size_t)N * (K / 64) * 2 * sizeof(half_t);
}

EAGLE_EXPORT int eagle_qmm_tile_w4g64(const uint32_t* wq, const void* scales, const void* biases, uint32_t* wt,
                                      void* sbt, int N, int K, int group_size, int bits, eagle_stream_t stream) {
  if (!wq || !scales || !biases || !wt || !sbt) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (N < 32 || (N % 32) != 0 || K < 512 || (K % 512) != 0) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(wq) || !eagle_aligned16(scales) || !eagle_aligned16(biases) || !eagle_aligned16(wt) ||
      !eagle_aligned16(sbt))
    return EAGLE_ERR_ALIGN;
  if (wt == wq || sbt == scales || sbt == biases) return EAGLE_ERR_SHAPE;    // not in place
  const long G = K / 64;
  const long total = (long)(N / 32) * G * 64 + (long)(N / 32) * (G / 8) * 64;
  hipLaunchKernelGGL(tile_weights_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), wq, static_cast<const half_t*>(scales),
                     static_cast<const half_t*>(biases), wt, static_cast<half_t*>(sbt), N, K);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmm_slab_partial_tiled_w4g64(const void* x, const uint32_t* wt, const void* sbt,
                                                    float* partial, size_t partial_bytes, int M, int N, int K,
                                                    int steps_per_slab, int small_scales, eagle_stream_t stream) {
  if (!x || !wt || !sbt || !partial) return EAGLE_ERR_NULL;
  if (!eagle_qmm_tiled_supported(M, N, K)) return EAGLE_ERR_SHAPE;
  const int slabs = eagle_qmm_slab_count(K, steps_per_slab);
  if (slabs < 1 || slabs > 65535) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wt) || !eagle_aligned16(sbt) || !eagle_aligned16(partial))
    return EAGLE_ERR_ALIGN;
  if (partial_bytes < eagle_qmm_slab_partial_bytes_rows(M, N, K, steps_per_slab)) return EAGLE_ERR_WORKSPACE;
  const int mr = M > SLAB_ROWS ? 2 : 1;
  const int bufs = steps_per_slab > SLAB_RING ? 2 : 1;
  const size_t lds = (size_t)bufs * mr * SLAB_XBUF * sizeof(half_t);
  static bool configured = false;
  if (!configured) {
    const int most = 2 * SLAB_XBUF * (int)sizeof(half_t);
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 1, false, 4, 1, true, false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 1, false, 4, 1, true, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 2, false, 4, 1, true, false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 2, false, 4, 1, true, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) != hipSuccess)
      return EAGLE_ERR_HIP;
    configured = true;
  }
  const dim3 grid((N + 127) / 128, slabs);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const half_t* xh = static_cast<const half_t*>(x);
  const half_t* sb = static_cast<const half_t*>(sbt);
#define EAGLE_TL_PARTIAL(MRV, SUB)                                                                         \
  hipLaunchKernelGGL((qmm_slab_w4g64_kernel<false, MRV, false, 4, 1, true, SUB>), grid, dim3(256), lds, st, xh, wt, \
                     sb, (const half_t*)nullptr, partial, M, N, K, steps_per_slab, bufs)
  if (mr == 2) {
    if (small_scales) EAGLE_TL_PARTIAL(2, true); else EAGLE_TL_PARTIAL(2, false);
  } else {
    if (small_scales) EAGLE_TL_PARTIAL(1, true); else EAGLE_TL_PARTIAL(1, false);
  }
#undef EAGLE_TL_PARTIAL
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmm_slab_swiglu_tiled_w4g64_f16(const void* x, const uint32_t* wt, const void* sbt,
                                                       const void* bias, void* out, int M, int N, int K,
                                                       int small_scales, eagle_stream_t stream) {
  if (!x || !wt || !sbt || !out) return EAGLE_ERR_NULL;
  if (!eagle_qmm_tiled_supported(M, N, K)) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wt) || !eagle_aligned16(sbt) || !eagle_aligned16(out) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  const int steps = K / 64;                      // one slab over all of K
  // the two K sizes of the benchmark targets go to the kernel with two waves per weight tile
  if (M <= SLAB_ROWS && (steps == 56 || steps == 64)) {
    hipStream_t bst = static_cast<hipStream_t>(stream);
    const half_t* xh = static_cast<const half_t*>(x);
    const half_t* sb = static_cast<const half_t*>(sbt);
    const half_t* bh = static_cast<const half_t*>(bias);
    half_t* oh = static_cast<half_t*>(out);
    if (steps == 56)
      return small_scales ? launch_burst<5, true, true, 7, 7>(xh, wt, sb, nullptr, nullptr, M, N, K, steps, 1, bh, oh, bst)
                          : launch_burst<5, true, false, 7, 7>(xh, wt, sb, nullptr, nullptr, M, N, K, steps, 1, bh, oh, bst);
    return small_scales ? launch_burst<4, true, true, 8, 8>(xh, wt, sb, nullptr, nullptr, M, N, K, steps, 1, bh, oh, bst)
                        : launch_burst<4, true, false, 8, 8>(xh, wt, sb, nullptr, nullptr, M, N, K, steps, 1, bh, oh, bst);
  }
  const int mr = M > SLAB_ROWS ? 2 : 1;
  int nwv = 4;
  while (nwv < 8 && (N + 32 * nwv - 1) / (32 * nwv) > NUM_CU) nwv += (nwv == 6 ? 2 : 1);
  const int blocks = (N + 32 * nwv - 1) / (32 * nwv);
  const int bufs = steps > SLAB_RING && !(mr == 2 && blocks > NUM_CU) ? 2 : 1;   // as the row-major form
  const size_t lds = (size_t)bufs * mr * SLAB_XBUF * sizeof(half_t);
  static bool configured = false;
  if (!configured) {
    const int most = 2 * SLAB_XBUF * (int)sizeof(half_t);
    bool ok = true;
#define EAGLE_TL_SWI_ATTR(NW)                                                                                    \
  ok = ok &&                                                                                                     \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 1, true, NW, 2, true, false>), \
                           hipFuncAttributeMaxDynamicSharedMemorySize, most) == hipSuccess &&                    \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 1, true, NW, 2, true, true>),  \
                           hipFuncAttributeMaxDynamicSharedMemorySize, most) == hipSuccess &&                    \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 2, true, NW, 1, true, false>), \
                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) == hipSuccess &&                \
       hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_slab_w4g64_kernel<false, 2, true, NW, 1, true, true>),  \
                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * most) == hipSuccess
    EAGLE_TL_SWI_ATTR(4);
    EAGLE_TL_SWI_ATTR(5);
    EAGLE_TL_SWI_ATTR(6);
    EAGLE_TL_SWI_ATTR(8);
#undef EAGLE_TL_SWI_ATTR
    if (!ok) return EAGLE_ERR_HIP;
    configured = true;
  }
  const dim3 grid(blocks, 1);
  hipStream_t st = static_cast<hipStream_t>(stream);
#define EAGLE_TL_SWI_LAUNCH(NW, MRV, SUB)                                                                \
  hipLaunchKernelGGL((qmm_slab_w4g64_kernel<false, MRV, true, NW, (MRV == 1 ? 2 : 1), true, SUB>), grid,  \
                     dim3(64 * NW), lds, st, static_cast<const half_t*>(x), wt,                          \
                     static_cast<const half_t*>(sbt), (const half_t*)nullptr, (float*)nullptr, M, N, K,  \
                     steps, bufs, static_cast<const half_t*>(bias), static_cast<half_t*>(out))
#define EAGLE_TL_SWI_NW(NW)                                                                              \
  if (mr == 2) {                                                                                         \
    if (small_scales) EAGLE_TL_SWI_LAUNCH(NW, 2, true); else EAGLE_TL_SWI_LAUNCH(NW, 2, false);          \
  } else {                                                                                               \
    if (small_scales) EAGLE_TL_SWI_LAUNCH(NW, 1, true); else EAGLE_TL_SWI_LAUNCH(NW, 1, false);          \
  }
  switch (nwv) {
    case 4: EAGLE_TL_SWI_NW(4) break;
    case 5: EAGLE_TL_SWI_NW(5) break;
    case 6: EAGLE_TL_SWI_NW(6) break;
    default: EAGLE_TL_SWI_NW(8) break;
  }
#undef EAGLE_TL_SWI_NW
#undef EAGLE_TL_SWI_LAUNCH
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmm_rows_tiled_supported(int M, int N, int K) {
  return M >= 1 && M <= SLAB_ROWS && N >= 32 && (N % 32) == 0 && K >= 512 && (K % 512) == 0 && K <= 65536;
}

EAGLE_EXPORT int eagle_qmm_rows_tiled_w4g64_f16(const void* x, const uint32_t* wt, const void* sbt, const void* bias,
                                                void* out, int M, int N, int K, int small_scales,
                                                eagle_stream_t stream) {
  if (!x || !wt || !sbt || !out) return EAGLE_ERR_NULL;
  if (!eagle_qmm_rows_tiled_supported(M, N, K)) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wt) || !eagle_aligned16(sbt) || !eagle_aligned16(out) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  if (x == out) return EAGLE_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const half_t* xh = static_cast<const half_t*>(x);
  const half_t* sb = static_cast<const half_t*>(sbt);
  const half_t* bh = static_cast<const half_t*>(bias);
  half_t* oh = static_cast<half_t*>(out);
  // ten streaming waves (twenty tiles per workgroup) unless eight give a launch that still fits
  // one workgroup per compute unit and fills more of them
  const int tiles = N >> 5;
  const bool eight = (tiles + 15) / 16 <= NUM_CU;
  if (eight)
    return small_scales ? launch_rows_tiled<8, true>(xh, wt, sb, bh, oh, M, N, K, st)
                        : launch_rows_tiled<8, false>(xh, wt, sb, bh, oh, M, N, K, st);
  return small_scales ? launch_rows_tiled<10, true>(xh, wt, sb, bh, oh, M, N, K, st)
                      : launch_rows_tiled<10, false>(xh, wt, sb, bh, oh, M, N, K, st);
}

static int gemm_dispatch(const void* x, const uint32_t* wq, const void* scales, const void* biases,
                         const void* bias, void* out, int M, int N, int K, int group_size, int bits,
                         bool swiglu, eagle_stream_t stream) {
  if (!x || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  if (M < 1 || N < 8 || (N % 8) != 0 || K < 64 || (K % 64) != 0) return EAGLE_ERR_SHAPE;
  if (swiglu && (N % 32) != 0) return EAGLE_ERR_SHAPE;
  if ((long)M * K >= (1L << 31)) return EAGLE_ERR_SHAPE;      // the kernel indexes x with 32 bits
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(out) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 7u)))
    return EAGLE_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const half_t* xh = static_cast<const half_t*>(x);
  const half_t* sh = static_cast<const half_t*>(scales);
  const half_t* bh = static_cast<const half_t*>(biases);
  const half_t* bi = static_cast<const half_t*>(bias);
  half_t* oh = static_cast<half_t*>(out);
  // Block shape: 64 x 128, 128 x 128 or 128 x 256 (x rows x weight rows).  The compute unit with
  // the most workgroups sets the time, and a workgroup's work goes with its block (bigger
  // blocks do a little less per output: 0.55 / 1 / 1.85); the estimate below reproduced the
  // faster choice for every projection shape of the 7B / 8B / 0.5B models at 512 and 2048 rows.
  auto most = [](long blocks) { return (double)((blocks + NUM_CU - 1) / NUM_CU); };
  const long nb = (N + 127) / 128;
  const double cost_norm = most(nb * ((M + 127) / 128));
  const double cost_small = M > 64 ? 0.55 * most(nb * ((M + 63) / 64)) : 1e30;
  const double cost_big = 1.85 * most(((N + 255) / 256) * (long)((M + 127) / 128));
  const bool small = cost_small < cost_norm && cost_small <= cost_big;
  const bool big = !small && cost_big < cost_norm;
  // scales and biases per fetch: as many groups as divide a row and as the base addresses are
  // aligned for
  const uintptr_t sb_addr = reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases);
  const int sbw = (K % 512) == 0 && (sb_addr & 15u) == 0 ? 8
                : (K % 256) == 0 && (sb_addr & 7u) == 0  ? 4
                : (K % 128) == 0 && (sb_addr & 3u) == 0  ? 2
                                                         : 1;
#define EAGLE_GEMM_SHAPE(NTW, MT)                                                              \
  switch (sbw) {                                                                               \
    case 8: return launch_gemm<NTW, MT, 8>(xh, wq, sh, bh, bi, oh, M, N, K, st);               \
    case 4: return launch_gemm<NTW, MT, 4>(xh, wq, sh, bh, bi, oh, M, N, K, st);               \
    case 2: return launch_gemm<NTW, MT, 2>(xh, wq, sh, bh, bi, oh, M, N, K, st);               \
    default: return launch_gemm<NTW, MT, 1>(xh, wq, sh, bh, bi, oh, M, N, K, st);              \
  }
  // two K groups per workgroup where the grid would leave a compute unit with one workgroup
  const long wgs = small ? nb * ((M + 63) / 64) : big ? ((N + 255) / 256) * (long)((M + 127) / 128) : nb * ((M + 127) / 128);
  if (swiglu) {
    // the wide gate|up matrix: the 128 x 256 block where it pays, else 128 x 128
    switch (sbw) {
      case 8: return big ? launch_gemm<2, 4, 4, 1, true>(xh, wq, sh, bh, bi, oh, M, N, K, st)
                         : launch_gemm<1, 4, 8, 1, true>(xh, wq, sh, bh, bi, oh, M, N, K, st);
      case 4: return launch_gemm<1, 4, 4, 1, true>(xh, wq, sh, bh, bi, oh, M, N, K, st);
      case 2: return launch_gemm<1, 4, 2, 1, true>(xh, wq, sh, bh, bi, oh, M, N, K, st);
      default: return launch_gemm<1, 4, 1, 1, true>(xh, wq, sh, bh, bi, oh, M, N, K, st);
    }
  }
  const bool split_k = sbw == 8 && (K % 1024) == 0 && wgs <= GEMM_SPLIT_WGS;
  if (split_k) {
    if (small) return launch_gemm<1, 2, 8, 2>(xh, wq, sh, bh, bi, oh, M, N, K, st);
    if (!big) return launch_gemm<1, 4, 8, 2>(xh, wq, sh, bh, bi, oh, M, N, K, st);
  }
  if (small) { EAGLE_GEMM_SHAPE(1, 2) }
  // (the 128 x 256 block takes its scales four groups per fetch at most: with eight it spills
  // twenty registers and is no faster, 149-153 us against 143-152 us for 512 x 28672 x 4096)
  if (big && sbw == 8) return launch_gemm<2, 4, 4>(xh, wq, sh, bh, bi, oh, M, N, K, st);
  if (big) { EAGLE_GEMM_SHAPE(2, 4) }
  EAGLE_GEMM_SHAPE(1, 4)
#undef EAGLE_GEMM_SHAPE
}

EAGLE_EXPORT int eagle_qmm_gemm_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                          const void* biases, const void* bias, void* out, int M, int N,
                                          int K, int group_size, int bits, eagle_stream_t stream) {
  return gemm_dispatch(x, wq, scales, biases, bias, out, M, N, K, group_size, bits, false, stream);
}

EAGLE_EXPORT int eagle_qmm_gemm_swiglu_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                                 const void* biases, const void* bias, void* out, int M,
                                                 int N, int K, int group_size, int bits,
                                                 eagle_stream_t stream) {
  return gemm_dispatch(x, wq, scales, biases, bias, out, M, N, K, group_size, bits, true, stream);
}
