// Tree-masked grouped-query attention of 32 query tokens per piece against a KV cache (gfx950).
//
//   out[t, h*hd + d] = sum_j softmax_j( scale * q[h,t,:] . k[g,j,:] + mask[t,j] ) v[g,j,d]
//
// The first P = *cache_len_dev cache rows are the prefix, visible to every tree token;
// rows P .. P+T-1 are the tree tokens, token j visible to token i iff bit j of
// tree_mask_bits[i] is set (the ancestor-or-self mask of mlx_eagle.py:239-248,337-338).
// Call site replaced: mlx_llama.py:185-195.
//
// Split-KV: grid (kv head g, key split s); one wave per query head of the group, so a
// K/V tile is read from memory once per group and shared through LDS.  Per block of 32 keys
// (a tile holds one or two) a
// wave computes S^T = K Q^T with v_mfma_f32_32x32x16_f16 (rows = keys, columns = the 32
// tree tokens), runs the online softmax on its accumulator (a lane owns one tree token,
// its partner lane+32 the other half of the keys), and feeds exp(S^T) straight back as
// the B operand of O^T += V^T P^T; only V needs a transposed read from LDS
// (ds_read_b64_tr_b16).  Partial (m, l, O) per split go to a workspace and a second kernel
// merges them.  The key tiles of the live length are dealt evenly to as many splits as give
// each at least two tiles and the launch at most as many workgroups as the GPU holds at once;
// the busiest workgroup sets the time.
//
// More than 32 query rows go in pieces of 32 on blockIdx.z, one launch pair for all pieces: the
// pieces of a causal prompt chunk (mlx_llama.py:275-276; each with its own cache length, the
// mask generated in the kernel) or of a tree of up to 64 tokens (one length, two mask words per
// query).
//
// The draft-side form (mlx_eagle.py:143-178,207) has fewer query rows than masked key rows: T
// queries see the P prefix rows and, through masks of one or two 32-bit words per query, the
// Tk <= 64 rows P .. P+Tk-1 written by the earlier expansion levels and this one.
#include "common.h"

#include <math.h>

namespace {

constexpr int KT = 32;   // keys per tile
constexpr float M_FLOOR = -3.0e38f;   // running maximum of a row that has seen no key yet

// ds_read_b64_tr_b16: 16 lanes x 4 halves, transposed (lane i of a group of 16 receives element
// i % 4 of the lanes 4 j + i / 4, j = 0..3 of the group); the address is 8-byte aligned
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
__device__ inline half4_t lds_read_tr16(const unsigned char* p) {
  const fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t*)(p));
  return __builtin_bit_cast(half4_t, v);
}

// splits that get work when `ntiles` key tiles are dealt to a grid of `nsplit` splits
// `lanes` = KV groups x pieces of query rows, the (group, piece) pairs that share the GPU: with
// many of them (a prompt chunk) the keys are split less, so that the launch has about as many
// workgroups as the GPU holds at once (`slots`) and each covers more tiles per partial result
// it writes (8B shape, 512-row chunk, us per launch pair with 2 / 4 / 8 / 16 tiles at least: 33 /
// 29 / 33 / 44 on an empty cache, 94 / 78 / 70 / 66 behind 1536 rows).
__host__ __device__ inline int active_splits(int ntiles, int nsplit, int lanes, int slots, int floor_tiles) {
  int tpw = (ntiles + nsplit - 1) / nsplit;
  int min_tiles = (lanes * ntiles + slots - 1) / slots;
  if (min_tiles < floor_tiles) min_tiles = floor_tiles;
  if (tpw < min_tiles) tpw = min_tiles;
  return (ntiles + tpw - 1) / tpw;
}

// Workgroups of `rep` waves that the 256 compute units hold at once: the split kernel's registers
// allow two waves per SIMD at head dimension 128 and three at 64.  One workgroup more than that
// costs a second round (a tree of 40 tokens at seven heads per group: 264 workgroups, 20.6 us;
// 176 workgroups, one round).
__host__ __device__ inline int split_slots(int rep, int hd) {
  const int waves_per_cu = hd > 64 ? 8 : 12;
  const int per_cu = waves_per_cu / rep;
  return 256 * (per_cu < 1 ? 1 : per_cu);
}

// q [H,T,hd] is rotated already and the cache holds the tree rows.
// NVU: 16-byte vectors of a K (or V) tile per thread, a power of two with NVU * blockDim.x >= the
// vectors of a tile.  DEPTH: tiles requested ahead, each in registers of its own (a tile's way
// from the L2 into LDS takes longer than its arithmetic: with one tile ahead the loop runs at one
// load latency per tile).
template <int V>
struct Stage { static constexpr int value = V; };

// SUB: 32-key blocks per tile (1 or 2).  With two, the S products, the exponentials and the O
// products of 64 keys each form one phase of a tile instead of two: the phases of a tile depend on
// each other inside a wave, so a tile of 64 keys takes little longer than one of 32.
template <int HD, bool WIDE, int NVU, int DEPTH, int SUB>
__global__ __launch_bounds__(512) void tree_attn_split_kernel(
    const half_t* __restrict__ q, half_t* kc, half_t* vc,
    const uint32_t* __restrict__ mask_bits, const int32_t* __restrict__ len_dev,
    half_t* __restrict__ part_o, float* __restrict__ part_ml, int T, int H, int G, long cap,
    float scale_log2e, int Tk, int q_rows, int len_stride) {
  constexpr int KSTEPS = HD / 16;       // MFMA steps over the head dimension for S
  constexpr int DB = HD / 32;           // 32-wide blocks of the head dimension for O
  constexpr int STR = HD * 2 + 16;      // LDS row stride in bytes (pad: conflict-free reads)
  constexpr int VEC_ROW = HD / 8;       // 16-byte vectors per K/V row
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  constexpr int KTT = KT * SUB;         // keys per tile
  unsigned char* ldsK = lds;
  unsigned char* ldsV = lds + KTT * STR;

  const int g = blockIdx.x;
  const int split = blockIdx.y;
  const int nsplit = gridDim.y;
  const int rep = H / G;
  const int tid = threadIdx.x;
  const int nthr = blockDim.x;          // rep * 64
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int ql = lane & 31;             // tree token (column of S^T / O^T)
  const int hb = lane >> 5;             // which half of the k / key index this lane holds
  const int head = g * rep + wave;

  // blockIdx.z: piece of 32 query rows, queries at rows 32 * piece of q [H, q_rows, hd] (the last
  // piece may hold fewer).  The pieces of a causal pass have a cache length each (len_stride 1),
  // those of a tree of more than 32 tokens share one length and the masked rows (len_stride 0,
  // mask words of query row 32 * piece + ql); a single piece otherwise.
  // (the last piece of a causal pass sees the most keys: dispatched first)
  const int piece = gridDim.z - 1 - blockIdx.z;
  const int qrow = piece * 32 + (lane & 31);
  if (T > q_rows - piece * 32) T = q_rows - piece * 32;
  int P = len_dev[piece * len_stride];
  // never index past the cache, whatever the counter says (a graph replayed beyond the
  // capacity would otherwise read beyond the last head's buffer)
  if (P > cap - Tk) P = (int)(cap - Tk);
  if (P < 0) P = 0;
  const int Ltot = P + Tk;                // Tk = T unless WIDE
  const int ntiles = (Ltot + KTT - 1) / KTT;
  // Splits in use for this length: every workgroup gets at most `tpw` key tiles, two at
  // least (with one, writing and merging the partials costs more than reading the keys).
  // The tile count of the busiest workgroup sets the time, so the tiles are spread evenly
  // over exactly as many workgroups as that takes; the rest of the grid leaves at once.
  const int nactive = active_splits(ntiles, nsplit, gridDim.x * gridDim.z, split_slots(rep, HD), 3 - SUB);
  if (split >= nactive) return;
  half8_t qreg[KSTEPS];
#pragma unroll
  for (int kk = 0; kk < KSTEPS; ++kk) {
    qreg[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (ql < T) {
      const half_t* qp = q + ((long)head * q_rows + qrow) * HD;
      qreg[kk] = *reinterpret_cast<const half8_t*>(qp + kk * 16 + hb * 8);
    }
  }
  // WIDE: two mask words per query (masked key rows 0..31 and 32..63)
  // no mask array: causal among the T rows
  const uint32_t mybits = ql < T ? (mask_bits ? mask_bits[WIDE ? 2 * qrow : ql] : (2u << ql) - 1u) : 0u;
  const uint32_t mybits_hi = (WIDE && ql < T && mask_bits) ? mask_bits[2 * qrow + 1] : 0u;

  float m_run = M_FLOOR, l_run = 0.f;
  // this lane's address for the transposing loads of V (see the O^T step below)
  const unsigned char* vt_base =
      ldsV + (4 * hb + ((lane & 15) >> 2)) * STR + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  float16_t o_acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[db][i] = 0.f;

  const half_t* kbase_ptr = kc + (long)g * cap * HD;
  const half_t* vbase_ptr = vc + (long)g * cap * HD;

  // This workgroup's tiles are split, split + nactive, ...: all workgroups share the live part
  // of the cache however short it is.  The next DEPTH tiles are in flight into registers while
  // the current one is being used.
  constexpr int NVEC = KTT * VEC_ROW;                // 16-byte vectors per K (or V) tile
  half8_t kreg[DEPTH][NVU], vreg[DEPTH][NVU];
  auto fetch = [&](auto S, int tile) {
    constexpr int st = decltype(S)::value;
    const int kb = tile * KTT;
#pragma unroll
    for (int it = 0; it < NVU; ++it) {
      int v = tid + it * nthr;
      if (v > NVEC - 1) v = NVEC - 1;
      const int row = v / VEC_ROW;
      const int c = v % VEC_ROW;
      int kidx = kb + row;
      if (kidx > Ltot - 1) kidx = Ltot - 1;          // rows past the end are masked out below
      const half_t* kp = kbase_ptr + (long)kidx * HD;
      const half_t* vp = vbase_ptr + (long)kidx * HD;
      kreg[st][it] = *reinterpret_cast<const half8_t*>(kp + c * 8);
      vreg[st][it] = *reinterpret_cast<const half8_t*>(vp + c * 8);
    }
  };
  auto stash = [&](auto S) {
    constexpr int st = decltype(S)::value;
#pragma unroll
    for (int it = 0; it < NVU; ++it) {
      const int v = tid + it * nthr;
      if (v < NVEC) {
        const int row = v / VEC_ROW;
        const int c = v % VEC_ROW;
        *reinterpret_cast<half8_t*>(ldsK + row * STR + c * 16) = kreg[st][it];
        *reinterpret_cast<half8_t*>(ldsV + row * STR + c * 16) = vreg[st][it];
      }
    }
  };

  // Every fetch is issued whether or not its tile exists (the index is clamped to the last
  // tile, whose rows are in the cache): with a fetch under a condition the compiler no longer
  // knows how many loads are outstanding where a stage is waited for, and waits for all of them.
  auto tile_at = [&](int t) { return t < ntiles ? t : ntiles - 1; };
  // (and the stages are requested in the order in which they are waited for, here as in the loop)
  __builtin_amdgcn_sched_barrier(0);
  fetch(Stage<0>{}, split);
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (DEPTH > 1) fetch(Stage<1>{}, tile_at(split + nactive));
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (DEPTH > 2) fetch(Stage<2>{}, tile_at(split + 2 * nactive));
  __builtin_amdgcn_sched_barrier(0);
  // one tile: its registers (stage S) into LDS, the tile DEPTH ahead requested into the same
  // registers, then the arithmetic on LDS
  auto do_tile = [&](auto S, int tile) {
    constexpr int st = decltype(S)::value;
    const int kb = tile * KTT;
    __syncthreads();   // every wave is done with the previous tile
    stash(S);
    fetch(S, tile_at(tile + DEPTH * nactive));
    __syncthreads();

    // S^T[key][token] = sum_d K[key][d] Q[token][d], one accumulator per block of 32 keys
    float16_t sacc[SUB];
#pragma unroll
    for (int h = 0; h < SUB; ++h)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[h][i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
#pragma unroll
      for (int h = 0; h < SUB; ++h) {
        const half8_t a = *reinterpret_cast<const half8_t*>(ldsK + (32 * h + ql) * STR + kk * 32 + hb * 16);
        sacc[h] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[kk], sacc[h], 0, 0, 0);
      }

    // accumulator register i of this lane is key 8*(i/4) + 4*hb + i%4 of its block.  The scores
    // stay unscaled: the scale (> 0) goes into the exponent's fused multiply-add, and the running
    // maximum starts at a finite floor instead of -inf, so that no case needs a select.
    float bm = M_FLOOR;
    if (kb + KTT <= P) {
      // a tile of prefix rows: visible to every token, no mask arithmetic
#pragma unroll
      for (int h = 0; h < SUB; ++h)
#pragma unroll
        for (int i = 0; i < 16; ++i) bm = fmaxf(bm, sacc[h][i]);
    } else {
#pragma unroll
      for (int h = 0; h < SUB; ++h)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kb + 32 * h + 8 * (i >> 2) + 4 * hb + (i & 3);
          const int rel = key - P;
          const uint32_t word = (WIDE && rel >= 32) ? mybits_hi : mybits;
          // (bitwise, not short-circuit: straight-line selects instead of a branch per key)
          const bool vis = (rel < 0) | ((key < Ltot) & (((word >> (rel & 31)) & 1u) != 0u));
          sacc[h][i] = vis ? sacc[h][i] : -INFINITY;
          bm = fmaxf(bm, sacc[h][i]);
        }
    }
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(m_run, bm * scale_log2e);
    // arguments are <= 0: the bare hardware exp2 (results below 2^-126 flush to zero, -inf gives 0)
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float psum = 0.f;
    half8_t bp[SUB][2];     // exp(S^T) as the B operand of the O products: step u = registers 8u..8u+7
#pragma unroll
    for (int h = 0; h < SUB; ++h)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = __builtin_amdgcn_exp2f(fmaf(sacc[h][i], scale_log2e, -m_new));
        psum += pv;
        bp[h][i >> 3][i & 7] = (half_t)pv;
      }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (alpha != 1.f) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[db][i] *= alpha;
    }

    // O^T[d][token] += sum_key V[key][d] P[token][key]; step u of block h covers accumulator
    // registers 8u..8u+7, i.e. keys 32h + 8*(2u + j/4) + 4*hb + j%4, j = 0..7.  The V^T operand
    // comes from the row-major tile through the transposing LDS load: within 16 lanes, lane i
    // receives element i % 4 of the four lanes 4 jj + i / 4, so lane s of a group asks for key row
    // s / 4 at the four d columns 4 (s % 4) .. + 3 of the group's 16 and gets four keys of its own d.
#pragma unroll
    for (int h = 0; h < SUB; ++h)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const half4_t lo = lds_read_tr16(vt_base + (32 * h + 16 * u) * STR + db * 64);
          const half4_t hi = lds_read_tr16(vt_base + (32 * h + 16 * u + 8) * STR + db * 64);
          const half8_t a = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bp[h][u], o_acc[db], 0, 0, 0);
        }
  };
  // whole rounds of DEPTH tiles (no condition between the stages of a round, so that the loads
  // outstanding at every wait are known), then the last DEPTH - 1 tiles at most
  int t0 = split;
  for (; t0 + (DEPTH - 1) * nactive < ntiles; t0 += DEPTH * nactive) {
    do_tile(Stage<0>{}, t0);
    if constexpr (DEPTH > 1) do_tile(Stage<1>{}, t0 + nactive);
    if constexpr (DEPTH > 2) do_tile(Stage<2>{}, t0 + 2 * nactive);
  }
  if constexpr (DEPTH > 1) {
    if (t0 < ntiles) {
      do_tile(Stage<0>{}, t0);
      if constexpr (DEPTH > 2)
        if (t0 + nactive < ntiles) do_tile(Stage<1>{}, t0 + nactive);
    }
  }

  // partials: part_ml [H][nsplit][32][2], part_o [H][nsplit][32][HD]
  const long slot = (((long)piece * H + head) * nsplit + split) * 32 + ql;
  if (hb == 0) {
    part_ml[slot * 2 + 0] = m_run;
    part_ml[slot * 2 + 1] = l_run;
  }
  half_t* po = part_o + slot * HD;     // fp16: |O| <= keys per split, relative error 2^-11
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int d0 = db * 32 + 8 * i4 + 4 * hb;
      half4_t v = half4_t{(half_t)o_acc[db][4 * i4 + 0], (half_t)o_acc[db][4 * i4 + 1],
                          (half_t)o_acc[db][4 * i4 + 2], (half_t)o_acc[db][4 * i4 + 3]};
      *reinterpret_cast<half4_t*>(po + d0) = v;
    }
}

// Merge the splits.  Grid (H, T / 4): a workgroup owns four tree tokens of one head; one
// thread per four output elements.  The softmax weights of the splits are computed once per
// token with one split per lane, then every thread adds its slice of the partial outputs.
constexpr int MERGE_TOK = 4;

template <int HD>
__global__ void tree_attn_merge_kernel(const half_t* __restrict__ part_o,
                                       const float* __restrict__ part_ml,
                                       half_t* __restrict__ out, int T, int H, int nsplit,
                                       const int32_t* __restrict__ len_dev, long cap,
                                       int Tk, int q_rows, int len_stride, int groups, int sub) {
  const int piece = blockIdx.z;                     // as in the split kernel
  if (T > q_rows - piece * 32) T = q_rows - piece * 32;
  part_o += (long)piece * H * nsplit * 32 * HD;
  part_ml += (long)piece * H * nsplit * 32 * 2;
  out += (long)piece * 32 * H * HD;
  constexpr int QW = HD / 4;                       // threads per token
  constexpr int TPW = 256 / HD;                    // tokens per wave: MERGE_TOK tokens on HD / 64 waves
  constexpr int PRE = 32;                          // partial outputs requested before anything is waited for
  __shared__ float wts[MERGE_TOK][64];
  const int head = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // Everything that does not depend on the live length is requested first: the (m, l) pairs
  // of every split of the grid and the first partial outputs.  Splits beyond the active
  // ones hold stale values; they are masked (m) or skipped (O) below, never multiplied.
  float2_t ml[TPW];
#pragma unroll
  for (int k = 0; k < TPW; ++k) {
    int t = blockIdx.y * MERGE_TOK + wave * TPW + k;
    if (t > T - 1) t = T - 1;
    const int sp = lane < nsplit ? lane : nsplit - 1;
    ml[k] = *reinterpret_cast<const float2_t*>(part_ml + (((long)head * nsplit + sp) * 32 + t) * 2);
  }
  const int tl = tid / QW;
  const int dq = tid % QW;
  const int t = blockIdx.y * MERGE_TOK + tl;
  const int t_c = t < T ? t : T - 1;
  const half_t* src = part_o + ((long)head * nsplit * 32 + t_c) * HD + dq * 4;
  // One or two pieces of query rows (the tree step: most splits of the grid are active): every
  // split's partial output is requested before the length is known.  More pieces (a prompt
  // chunk: a few active splits out of a grid sized for the longest cache): only the active
  // ones, after it (8B shape, 16 pieces behind 1536 cache rows: 20 -> 9 us).
  const bool eager = gridDim.z <= 2;
  half4_t pre[PRE];
  if (eager) {
#pragma unroll
    for (int k = 0; k < PRE; ++k)
      if (k < nsplit) pre[k] = *reinterpret_cast<const half4_t*>(src + (long)k * 32 * HD);
  }

  int P = len_dev[piece * len_stride];
  if (P > cap - Tk) P = (int)(cap - Tk);    // as in the split kernel
  if (P < 0) P = 0;
  const int nact = active_splits((P + Tk + KT * sub - 1) / (KT * sub), nsplit, groups * gridDim.z,
                                 split_slots(H / groups, HD), 3 - sub);   // as in the split kernel
  if (!eager) {
#pragma unroll
    for (int k = 0; k < PRE; ++k)
      if (k < nact) pre[k] = *reinterpret_cast<const half4_t*>(src + (long)k * 32 * HD);
  }
#pragma unroll
  for (int k = 0; k < TPW; ++k) {
    const float m = lane < nact ? ml[k][0] : -INFINITY;
    const float l = lane < nact ? ml[k][1] : 0.f;
    const float mx = wave_max(m);
    const float w = m == -INFINITY ? 0.f : exp2f(m - mx);
    const float den = wave_sum(w * l);
    wts[wave * TPW + k][lane] = den > 0.f ? w / den : 0.f;
  }
  __syncthreads();
  if (t >= T) return;
  float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < PRE; ++k)
    if (k < nact) {
      const float wk = wts[tl][k];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += wk * (float)pre[k][e];
    }
  for (int s0 = PRE; s0 < nact; s0 += 8) {
    half4_t v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int sp = s0 + k < nact ? s0 + k : nact - 1;
      v[k] = *reinterpret_cast<const half4_t*>(src + (long)sp * 32 * HD);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (s0 + k < nact) {
        const float wk = wts[tl][s0 + k];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += wk * (float)v[k][e];
      }
  }
  half4_t o = half4_t{(half_t)acc[0], (half_t)acc[1], (half_t)acc[2], (half_t)acc[3]};
  *reinterpret_cast<half4_t*>(out + ((long)t * H + head) * HD + dq * 4) = o;
}

// Key splits of the grid (gridDim.y), sized for the longest length; how many of them get work
// follows the live length inside the kernels (active_splits).
int splits_for(int max_len, int G) {
  (void)G;
  const int ntiles = (max_len + KT - 1) / KT;
  int n = (ntiles + 1) / 2;            // two tiles per workgroup at the longest length
  if (n > 64) n = 64;                  // one split per lane in the merge
  if (n < 1) n = 1;
  return n;
}

template <int HD, bool WIDE = false>
int launch_attention(const half_t* q, half_t* kc, half_t* vc, const uint32_t* bits, const int32_t* len,
                     void* out, int T, int H, int G, long cap, int max_len, float scale, void* workspace,
                     hipStream_t st,
                     int Tk = 0, int pieces = 1, int q_rows = 0, int len_stride = 1) {
  if (!WIDE) Tk = T;
  if (q_rows == 0) q_rows = pieces * T;
  // The grid holds as many splits as the longest length makes active: a workgroup without
  // work still takes a slot for the 2 us in which it learns that from the cache length, and
  // thousands of them ahead of the last pieces' workgroups (a chunk of 16 pieces in a grid of 36
  // splits for 4 active ones) held those back by 18 of 44 us.
  const int rep = H / G;
  // 64 keys per tile where a tile's 16-byte vectors are at most four per thread (three or more
  // waves per workgroup at head dimension 128, two or more at 64), 32 keys otherwise
  const int need64 = (2 * KT * (HD / 8) + rep * 64 - 1) / (rep * 64);
  const int sub = need64 <= 4 ? 2 : 1;
  const int ktt = KT * sub;
  int nsplit = splits_for(max_len, G);
  nsplit = active_splits((max_len + ktt - 1) / ktt, nsplit, G * pieces, split_slots(rep, HD), 3 - sub);
  float* part_ml = static_cast<float*>(workspace);
  half_t* part_o = reinterpret_cast<half_t*>(part_ml + (size_t)pieces * H * nsplit * 32 * 2);
  const float sl2 = scale * 1.4426950408889634f;
  const size_t lds = 2 * ktt * (HD * 2 + 16);
  // vectors of a tile per thread (a power of two) and the tiles in flight that its registers allow
  const int need = (ktt * (HD / 8) + rep * 64 - 1) / (rep * 64);
#define EAGLE_ATTN_SPLIT(NVU, DEPTH, SUB)                                                                \
  hipLaunchKernelGGL((tree_attn_split_kernel<HD, WIDE, NVU, DEPTH, SUB>),                                \
                     dim3(G, nsplit, pieces), dim3(rep * 64), lds, st, q, kc, vc, bits, len, part_o, part_ml, T, \
                     H, G, cap, sl2, Tk, q_rows, len_stride)
  if (sub == 2) {
    if (need <= 1) EAGLE_ATTN_SPLIT(1, 3, 2);
    else if (need <= 2) EAGLE_ATTN_SPLIT(2, 2, 2);
    else EAGLE_ATTN_SPLIT(4, 1, 2);
  } else {
    if (need <= 1) EAGLE_ATTN_SPLIT(1, 3, 1);
    else if (need <= 2) EAGLE_ATTN_SPLIT(2, 3, 1);
    else if (need <= 4) EAGLE_ATTN_SPLIT(4, 2, 1);
    else EAGLE_ATTN_SPLIT(8, 1, 1);
  }
#undef EAGLE_ATTN_SPLIT
  hipLaunchKernelGGL(tree_attn_merge_kernel<HD>, dim3(H, (T + MERGE_TOK - 1) / MERGE_TOK, pieces),
                     dim3(MERGE_TOK * HD / 4), 0, st, part_o, part_ml, (half_t*)out, T, H, nsplit,
                     len, cap, Tk, q_rows, len_stride, G, sub);
  return eagle_launch_status();
}

__global__ void rope_table_kernel(const int32_t* __restrict__ pos, const float* __restrict__ inv_freq,
                                  float scale, float* __restrict__ out, int T, int half) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * half) return;
  const int i = idx % half;
  const int t = idx / half;
  const float lf = scale * inv_freq[i];
  const float theta = lf * (float)pos[t];
  float sn, cs;
  sincosf(theta, &sn, &cs);
  out[2 * idx] = cs;
  out[2 * idx + 1] = sn;
}

}  // namespace

EAGLE_EXPORT size_t eagle_tree_attention_workspace_bytes(int H, int hd, int max_len) {
  if (H < 1 || hd < 1 || max_len < 1) return 0;
  return (size_t)H * 64 * 32 * (hd + 2) * sizeof(float);   // at most 64 key splits
}

EAGLE_EXPORT int eagle_tree_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                                          const uint32_t* tree_mask_bits,
                                          const int32_t* cache_len_dev, void* out, int T, int H,
                                          int G, int hd, long capacity, int max_len, float scale,
                                          void* workspace, size_t workspace_bytes,
                                          eagle_stream_t stream) {
  if (!q || !k_cache || !v_cache || !tree_mask_bits || !cache_len_dev || !out) return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE || H < 1 || G < 1 || (H % G) != 0 || (H / G) > 8 ||
      (hd != 64 && hd != 128) || max_len < T || max_len > capacity || !(scale > 0.f))
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) ||
      !eagle_aligned16(out))
    return EAGLE_ERR_ALIGN;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_tree_attention_workspace_bytes(H, hd, max_len))
    return EAGLE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the kernel only reads the caches in this form
  half_t* kc = const_cast<half_t*>(static_cast<const half_t*>(k_cache));
  half_t* vc = const_cast<half_t*>(static_cast<const half_t*>(v_cache));
  if (hd == 128)
    return launch_attention<128>((const half_t*)q, kc, vc, tree_mask_bits, cache_len_dev, out, T, H,
                                        G, capacity, max_len, scale, workspace, st);
  return launch_attention<64>((const half_t*)q, kc, vc, tree_mask_bits, cache_len_dev, out, T, H, G,
                                     capacity, max_len, scale, workspace, st);
}

EAGLE_EXPORT int eagle_draft_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                                           const uint32_t* mask_words, const int32_t* cache_len_dev,
                                           void* out, int T, int Tk, int H, int G, int hd,
                                           long capacity, int max_len, float scale, void* workspace,
                                           size_t workspace_bytes, eagle_stream_t stream) {
  if (!q || !k_cache || !v_cache || !mask_words || !cache_len_dev || !out) return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE || Tk < 1 || Tk > 2 * EAGLE_MAX_TREE || H < 1 || G < 1 ||
      (H % G) != 0 || (H / G) > 8 || (hd != 64 && hd != 128) || max_len < Tk || max_len > capacity || !(scale > 0.f))
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) ||
      !eagle_aligned16(out))
    return EAGLE_ERR_ALIGN;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_tree_attention_workspace_bytes(H, hd, max_len))
    return EAGLE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  half_t* kc = const_cast<half_t*>(static_cast<const half_t*>(k_cache));
  half_t* vc = const_cast<half_t*>(static_cast<const half_t*>(v_cache));
  if (hd == 128)
    return launch_attention<128, true>((const half_t*)q, kc, vc, mask_words, cache_len_dev, out, T,
                                              H, G, capacity, max_len, scale, workspace, st, Tk);
  return launch_attention<64, true>((const half_t*)q, kc, vc, mask_words, cache_len_dev, out, T, H,
                                           G, capacity, max_len, scale, workspace, st, Tk);
}

EAGLE_EXPORT size_t eagle_tree_attention_wide_workspace_bytes(int T, int H, int hd, int max_len) {
  if (T < 1 || T > EAGLE_MAX_TREE_SLOTS) return 0;
  return (size_t)((T + 31) / 32) * eagle_tree_attention_workspace_bytes(H, hd, max_len);
}

EAGLE_EXPORT int eagle_tree_attention_wide_f16(const void* q, const void* k_cache, const void* v_cache,
                                               const uint32_t* mask_words, const int32_t* cache_len_dev,
                                               void* out, int T, int Tk, int H, int G, int hd,
                                               long capacity, int max_len, float scale, void* workspace,
                                               size_t workspace_bytes, eagle_stream_t stream) {
  if (!q || !k_cache || !v_cache || !mask_words || !cache_len_dev || !out) return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE_SLOTS || Tk < 1 || Tk > EAGLE_MAX_TREE_SLOTS || H < 1 || G < 1 ||
      (H % G) != 0 || (H / G) > 8 || (hd != 64 && hd != 128) || max_len < Tk || max_len > capacity || !(scale > 0.f))
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) ||
      !eagle_aligned16(out))
    return EAGLE_ERR_ALIGN;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_tree_attention_wide_workspace_bytes(T, H, hd, max_len))
    return EAGLE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  half_t* kc = const_cast<half_t*>(static_cast<const half_t*>(k_cache));
  half_t* vc = const_cast<half_t*>(static_cast<const half_t*>(v_cache));
  // pieces of 32 query rows over the same Tk masked rows and one cache length
  const int pieces = (T + 31) / 32;
  const int rows = T < 32 ? T : 32;
  if (hd == 128)
    return launch_attention<128, true>((const half_t*)q, kc, vc, mask_words, cache_len_dev, out, rows,
                                              H, G, capacity, max_len, scale, workspace, st, Tk, pieces, T, 0);
  return launch_attention<64, true>((const half_t*)q, kc, vc, mask_words, cache_len_dev, out, rows, H,
                                           G, capacity, max_len, scale, workspace, st, Tk, pieces, T, 0);
}

EAGLE_EXPORT size_t eagle_causal_attention_workspace_bytes(int R, int H, int hd, int max_len) {
  if (R < 32 || (R % 32) != 0) return 0;
  return (size_t)(R / 32) * eagle_tree_attention_workspace_bytes(H, hd, max_len);
}

EAGLE_EXPORT int eagle_causal_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                                            const int32_t* piece_len_dev, void* out, int R, int H, int G,
                                            int hd, long capacity, int max_len, float scale,
                                            void* workspace, size_t workspace_bytes,
                                            eagle_stream_t stream) {
  if (!q || !k_cache || !v_cache || !piece_len_dev || !out) return EAGLE_ERR_NULL;
  if (R < 32 || (R % 32) != 0 || R > EAGLE_MAX_CHUNK || H < 1 || G < 1 || (H % G) != 0 ||
      (H / G) > 8 || (hd != 64 && hd != 128) || max_len < 32 || max_len > capacity || !(scale > 0.f))
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) ||
      !eagle_aligned16(out))
    return EAGLE_ERR_ALIGN;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_causal_attention_workspace_bytes(R, H, hd, max_len))
    return EAGLE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  half_t* kc = const_cast<half_t*>(static_cast<const half_t*>(k_cache));
  half_t* vc = const_cast<half_t*>(static_cast<const half_t*>(v_cache));
  // the two-word form of the kernel: it keeps the cache length inside the buffer
  if (hd == 128)
    return launch_attention<128, true>((const half_t*)q, kc, vc, nullptr, piece_len_dev, out, 32, H,
                                              G, capacity, max_len, scale, workspace, st, 32, R / 32);
  return launch_attention<64, true>((const half_t*)q, kc, vc, nullptr, piece_len_dev, out, 32, H, G,
                                           capacity, max_len, scale, workspace, st, 32, R / 32);
}

EAGLE_EXPORT int eagle_rope_table_f32(const int32_t* positions, const float* inv_freqs,
                                      float scaling_factor, int T, int half_dim, float* out,
                                      eagle_stream_t stream) {
  if (!positions || !inv_freqs || !out) return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_CHUNK || half_dim < 1) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(out)) return EAGLE_ERR_ALIGN;
  const int total = T * half_dim;
  hipLaunchKernelGGL(rope_table_kernel, dim3((total + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), positions, inv_freqs, scaling_factor, out, T,
                     half_dim);
  return eagle_launch_status();
}
