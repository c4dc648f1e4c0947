// One launch for the attention block of a tree-verification step (gfx950):
// rotary embedding of q and of the new keys, append of the new K/V rows to the cache,
// tree-masked grouped-query attention against prefix + tree rows, and the merge of the key
// splits.  Call sites replaced: mlx_llama.py:166-195 (rope of q/k, cache update, SDPA).
//
//   out[t, h*hd + d] = sum_j softmax_j( scale * rope(q)[h,t,:] . K[g,j,:] + mask[t,j] ) V[g,j,d]
//
// K/V rows j < P = *cache_len_dev come from the cache; rows P .. P+T-1 are the tree tokens and
// come straight from the projection output (keys rotated on the fly), so no workgroup ever
// reads a cache row that this launch writes.  The workgroups of the first query head of each
// KV group store the new rows into the cache.
//
// Grid: one workgroup per (query head, key split), four waves each.  Key tiles of 32 rows are
// dealt round-robin to splits and then to the waves of a workgroup; a wave keeps the whole
// online softmax state of its tiles in registers (S^T = K Q^T and O^T += V^T P^T with
// v_mfma_f32_32x32x16_f16, K rows loaded directly in operand layout, V transposed through a
// wave-private LDS tile).  The four waves merge through LDS, the workgroup stores one partial
// (m, l, O) and the last workgroup of a head to arrive merges the splits in split order, so
// the result does not depend on arrival order.  Workgroups that share K/V rows (the heads of
// a KV group working on the same split) get consecutive slots of one XCD, whose L2 then
// serves the repeats.
#include "common.h"

#include <math.h>

namespace {

constexpr int KT = 32;       // keys per tile
constexpr int WAVES = 4;     // waves per workgroup
constexpr int MAX_SPLITS = 64;

__device__ inline uint64_t ld_relaxed(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void st_relaxed(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// (lo, hi) = elements i0..i0+7 and i0+half..i0+half+7 of a head vector; cs = 8 (cos, sin) pairs
__device__ inline void rotate_pair(half8_t& lo, half8_t& hi, const float* cs) {
  float4_t c[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) c[k] = *reinterpret_cast<const float4_t*>(cs + 4 * k);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float co = c[j >> 1][(j & 1) * 2], sn = c[j >> 1][(j & 1) * 2 + 1];
    const float x1 = (float)lo[j], x2 = (float)hi[j];
    lo[j] = (half_t)(x1 * co - x2 * sn);
    hi[j] = (half_t)(x1 * sn + x2 * co);
  }
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

template <int HD>
__global__ __launch_bounds__(WAVES * 64) void tree_attn_rope_kernel(
    const half_t* __restrict__ q_lin, const half_t* __restrict__ k_lin,
    const half_t* __restrict__ v_lin, long ld, const float* __restrict__ rope_cs,
    half_t* __restrict__ kc, half_t* __restrict__ vc, const uint32_t* __restrict__ mask_bits,
    const int32_t* __restrict__ len_dev, unsigned* __restrict__ counters,
    float* __restrict__ part_ml, half_t* __restrict__ part_o, half_t* __restrict__ out, int T,
    int H, int G, long cap, int nsplit, float scale_log2e) {
  constexpr int KSTEPS = HD / 16;       // MFMA steps over the head dimension for S
  constexpr int HK = KSTEPS / 2;        // chunk kk pairs with chunk kk + HK under the rotation
  constexpr int HALF = HD / 2;
  constexpr int DB = HD / 32;           // 32-wide blocks of the head dimension for O
  constexpr int STR = HD * 2 + 16;      // LDS row stride of a V tile in bytes
  constexpr int VEC_ROW = HD / 8;       // 16-byte vectors per K/V row
  constexpr int NVV = KT * VEC_ROW / 64;  // V vectors per lane per tile
  constexpr int OSTR = HD + 4;          // floats per token row of a wave's O in LDS
  constexpr int DPT = HD / 8;           // output elements per thread in the merges
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int rep = H / G;
  // slot -> (KV group, split, head of the group): the rep heads of a (group, split) pair sit
  // on one XCD (workgroups go to the 8 XCDs round-robin by linear id)
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int pair = (slot / rep) * 8 + xcd;
  if (pair >= G * nsplit) return;
  const int r = slot % rep;
  const int g = pair / nsplit;
  const int split = pair % nsplit;
  const int head = g * rep + r;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int ql = lane & 31;             // tree token (column of S^T / O^T); key row for K loads
  const int hb = lane >> 5;             // which half of the k / key index this lane holds

  long P = *len_dev;
  if (P > cap - T) P = cap - T;         // never index past the cache, whatever the counter says
  if (P < 0) P = 0;
  const int Ltot = (int)P + T;
  const int ntiles = (Ltot + KT - 1) / KT;

  const half_t* kbase = kc + (long)g * cap * HD;
  const half_t* vbase = vc + (long)g * cap * HD;
  const half_t* klin = k_lin + (long)g * HD;
  const half_t* vlin = v_lin + (long)g * HD;

  // Two tiles in flight per wave: register sets A and B are refilled as soon as their tile
  // has been consumed.  Fetches are unconditional (a tile index past the end re-reads the
  // last rows, which stay in cache) so that the load counters can be waited on exactly.
  half8_t kregA[KSTEPS], vregA[NVV], kregB[KSTEPS], vregB[NVV];
  auto fetch = [&](int tile, half8_t (&kreg)[KSTEPS], half8_t (&vreg)[NVV]) {
    const int kb = tile * KT;
    int key = kb + ql;
    if (key > Ltot - 1) key = Ltot - 1;              // rows past the end are masked out below
    const half_t* kp = key < P ? kbase + (long)key * HD : klin + (long)(key - P) * ld;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
      kreg[kk] = *reinterpret_cast<const half8_t*>(kp + kk * 16 + hb * 8);
#pragma unroll
    for (int it = 0; it < NVV; ++it) {
      const int v = lane + it * 64;
      const int c = v % VEC_ROW;
      int k2 = kb + v / VEC_ROW;
      if (k2 > Ltot - 1) k2 = Ltot - 1;
      const half_t* vp = k2 < P ? vbase + (long)k2 * HD : vlin + (long)(k2 - P) * ld;
      vreg[it] = *reinterpret_cast<const half8_t*>(vp + c * 8);
    }
  };

  const int tile0 = split + nsplit * wave;
  const int tstep = nsplit * WAVES;
  fetch(tile0, kregA, vregA);
  fetch(tile0 + tstep, kregB, vregB);

  // q of this head in B-operand layout: lane (token ql, half hb) holds q[ql][kk*16 + hb*8 .. +7];
  // the cos/sin table goes to LDS once, so that no rotation below needs a global load
  half8_t qreg[KSTEPS];
  {
    const int tq = ql < T ? ql : T - 1;
    const half_t* qp = q_lin + (long)tq * ld + (long)head * HD;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
      qreg[kk] = *reinterpret_cast<const half8_t*>(qp + kk * 16 + hb * 8);
  }
  float* cs_lds = reinterpret_cast<float*>(lds + WAVES * KT * STR);      // [T][HALF][2]
  for (int v = tid; v < T * HALF / 2; v += WAVES * 64)
    *reinterpret_cast<float4_t*>(cs_lds + 4 * v) = *reinterpret_cast<const float4_t*>(rope_cs + 4 * v);
  __syncthreads();
  if (ql < T) {
#pragma unroll
    for (int kk = 0; kk < HK; ++kk)
      rotate_pair(qreg[kk], qreg[kk + HK], cs_lds + (ql * HALF + kk * 16 + hb * 8) * 2);
  } else {
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) qreg[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
  const uint32_t mybits = ql < T ? mask_bits[ql] : 0u;

  float m_run = -INFINITY, l_run = 0.f;
  float16_t o_acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[db][i] = 0.f;

  unsigned char* ldsV = lds + wave * (KT * STR);

  auto process = [&](int tile, half8_t (&kreg)[KSTEPS], half8_t (&vreg)[NVV]) {
    const int kb = tile * KT;
    if (kb + KT > P) {
      // the tile holds tree rows: rotate their keys; the first head of the group appends them
      const int key = kb + ql;
      const bool fresh = key >= P && key < Ltot;
      if (fresh) {
#pragma unroll
        for (int kk = 0; kk < HK; ++kk)
          rotate_pair(kreg[kk], kreg[kk + HK],
                      cs_lds + ((key - (int)P) * HALF + kk * 16 + hb * 8) * 2);
        if (r == 0) {
          half_t* dst = kc + ((long)g * cap + key) * HD;
#pragma unroll
          for (int kk = 0; kk < KSTEPS; ++kk)
            *reinterpret_cast<half8_t*>(dst + kk * 16 + hb * 8) = kreg[kk];
        }
      }
      if (r == 0) {
#pragma unroll
        for (int it = 0; it < NVV; ++it) {
          const int v = lane + it * 64;
          const int k2 = kb + v / VEC_ROW;
          if (k2 >= P && k2 < Ltot)
            *reinterpret_cast<half8_t*>(vc + ((long)g * cap + k2) * HD + (v % VEC_ROW) * 8) = vreg[it];
        }
      }
    }

    // S^T[key][token] = sum_d K[key][d] Q[token][d]
    float16_t sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kreg[kk], qreg[kk], sacc, 0, 0, 0);

    // V tile to this wave's LDS, then the registers are free for the next tile
#pragma unroll
    for (int it = 0; it < NVV; ++it) {
      const int v = lane + it * 64;
      *reinterpret_cast<half8_t*>(ldsV + (v / VEC_ROW) * STR + (v % VEC_ROW) * 16) = vreg[it];
    }
    fetch(tile + 2 * tstep, kreg, vreg);

    // accumulator register i of this lane is key 8*(i/4) + 4*hb + i%4 of the tile
    float sv[16];
    float bm = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb + 8 * (i >> 2) + 4 * hb + (i & 3);
      const int rel = key - (int)P;
      const bool vis = (key < P) || (key < Ltot && ((mybits >> (rel & 31)) & 1u));
      sv[i] = vis ? sacc[i] * scale_log2e : -INFINITY;
      bm = fmaxf(bm, sv[i]);
    }
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(m_run, bm);
    float alpha = 1.f;
    float psum = 0.f;
    float p[16];
    if (m_new == -INFINITY) {
#pragma unroll
      for (int i = 0; i < 16; ++i) p[i] = 0.f;
    } else {
      alpha = exp2f(m_run - m_new);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        p[i] = exp2f(sv[i] - m_new);
        psum += p[i];
      }
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

    // O^T[d][token] += sum_key V[key][d] P[token][key]; step u covers accumulator
    // registers 8u..8u+7, i.e. keys 8*(2u + j/4) + 4*hb + j%4, j = 0..7.
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      half8_t bp;
#pragma unroll
      for (int j = 0; j < 8; ++j) bp[j] = (half_t)p[8 * u + j];
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        half8_t a;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = 8 * (2 * u + (j >> 2)) + 4 * hb + (j & 3);
          a[j] = *reinterpret_cast<const half_t*>(ldsV + key * STR + (db * 32 + ql) * 2);
        }
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bp, o_acc[db], 0, 0, 0);
      }
    }
  };
  for (int tile = tile0; tile < ntiles; tile += 2 * tstep) {
    process(tile, kregA, vregA);
    if (tile + tstep < ntiles) process(tile + tstep, kregB, vregB);
  }

  // ---- merge the waves of this workgroup through LDS (the V tiles are dead by now)
  __syncthreads();
  float* ow = reinterpret_cast<float*>(lds);                     // [WAVES][32][OSTR]
  float* mlw = ow + WAVES * 32 * OSTR;                           // [WAVES][32][2]
  int* flag = reinterpret_cast<int*>(mlw + WAVES * 32 * 2);
  {
    float* mine = ow + (wave * 32 + ql) * OSTR;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = db * 32 + 8 * i4 + 4 * hb;
        *reinterpret_cast<float4_t*>(mine + d0) =
            float4_t{o_acc[db][4 * i4 + 0], o_acc[db][4 * i4 + 1], o_acc[db][4 * i4 + 2],
                     o_acc[db][4 * i4 + 3]};
      }
    if (hb == 0) {
      mlw[(wave * 32 + ql) * 2 + 0] = m_run;
      mlw[(wave * 32 + ql) * 2 + 1] = l_run;
    }
  }
  __syncthreads();
  const int t = tid >> 3;               // token of this thread in both merges
  const int d0 = (tid & 7) * DPT;       // its slice of the head dimension
  float acc[DPT];
  float m_wg = -INFINITY, l_wg = 0.f;
  {
#pragma unroll
    for (int w = 0; w < WAVES; ++w) m_wg = fmaxf(m_wg, mlw[(w * 32 + t) * 2]);
#pragma unroll
    for (int e = 0; e < DPT; ++e) acc[e] = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float mw = mlw[(w * 32 + t) * 2];
      const float e_w = mw == -INFINITY ? 0.f : exp2f(mw - m_wg);
      l_wg += e_w * mlw[(w * 32 + t) * 2 + 1];
      const float* src = ow + (w * 32 + t) * OSTR + d0;
#pragma unroll
      for (int e = 0; e < DPT; ++e) acc[e] += e_w * src[e];
    }
  }
  // partials: part_ml [H][nsplit][32][2] fp32 (m, l), part_o [H][nsplit][32][HD] fp16 holding
  // O / l, which is a convex combination of V rows and so cannot overflow fp16
  {
    const float inv_l = l_wg > 0.f ? 1.f / l_wg : 0.f;
#pragma unroll
    for (int e = 0; e < DPT; ++e) acc[e] *= inv_l;
    const long pslot = ((long)head * nsplit + split) * 32 + t;
    uint64_t* po = reinterpret_cast<uint64_t*>(part_o + pslot * HD + d0);
#pragma unroll
    for (int e4 = 0; e4 < DPT / 4; ++e4) {
      union { half4_t h; uint64_t u; } cv;
      cv.h = half4_t{(half_t)acc[4 * e4 + 0], (half_t)acc[4 * e4 + 1], (half_t)acc[4 * e4 + 2],
                     (half_t)acc[4 * e4 + 3]};
      st_relaxed(po + e4, cv.u);
    }
    if ((tid & 7) == 0) {
      union { float f[2]; uint64_t u; } cv;
      cv.f[0] = m_wg;
      cv.f[1] = l_wg;
      st_relaxed(reinterpret_cast<uint64_t*>(part_ml + pslot * 2), cv.u);
    }
  }

  // ---- the last workgroup of this head to arrive merges the splits, in split order
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's partial stores are done
  __syncthreads();
  if (tid == 0) {
    const unsigned old =
        __hip_atomic_fetch_add(&counters[head], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = old == (unsigned)(nsplit - 1);
    if (old == (unsigned)(nsplit - 1))
      __hip_atomic_store(&counters[head], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!*flag || t >= T) return;

  // all loads of up to MCH splits are in flight together; longer lists are folded chunk by
  // chunk with a running maximum
  constexpr int MCH = 16;
  const uint64_t* ml_src = reinterpret_cast<const uint64_t*>(part_ml + ((long)head * nsplit * 32 + t) * 2);
  const uint64_t* o_src = reinterpret_cast<const uint64_t*>(part_o + ((long)head * nsplit * 32 + t) * HD + d0);
  float mx = -INFINITY, den = 0.f;
#pragma unroll
  for (int e = 0; e < DPT; ++e) acc[e] = 0.f;
  for (int s0 = 0; s0 < nsplit; s0 += MCH) {
    uint64_t mlr[MCH], orw[MCH][DPT / 4];
#pragma unroll
    for (int k = 0; k < MCH; ++k) {
      const long sp = s0 + k < nsplit ? s0 + k : nsplit - 1;
      mlr[k] = ld_relaxed(ml_src + sp * 32);
#pragma unroll
      for (int e4 = 0; e4 < DPT / 4; ++e4) orw[k][e4] = ld_relaxed(o_src + sp * (32 * HD / 4) + e4);
    }
    float cm = mx;
#pragma unroll
    for (int k = 0; k < MCH; ++k) {
      union { uint64_t u; float f[2]; } ml;
      ml.u = mlr[k];
      if (s0 + k < nsplit) cm = fmaxf(cm, ml.f[0]);
    }
    if (cm == -INFINITY) continue;
    const float resc = exp2f(mx - cm);                 // 0 on the first chunk (mx = -inf)
    den *= resc;
#pragma unroll
    for (int e = 0; e < DPT; ++e) acc[e] *= resc;
    mx = cm;
#pragma unroll
    for (int k = 0; k < MCH; ++k)
      if (s0 + k < nsplit) {
        union { uint64_t u; float f[2]; } ml;
        ml.u = mlr[k];
        const float w = ml.f[0] == -INFINITY ? 0.f : exp2f(ml.f[0] - mx) * ml.f[1];
        den += w;
#pragma unroll
        for (int e4 = 0; e4 < DPT / 4; ++e4) {
          union { uint64_t u; half4_t h; } cv;
          cv.u = orw[k][e4];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[4 * e4 + e] += w * (float)cv.h[e];
        }
      }
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  half_t* dst = out + ((long)t * H + head) * HD + d0;
#pragma unroll
  for (int e8 = 0; e8 < DPT / 8; ++e8) {
    half8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (half_t)(acc[8 * e8 + e] * inv);
    *reinterpret_cast<half8_t*>(dst + 8 * e8) = o;
  }
}

// Key splits per head: at most one workgroup per compute unit (a workgroup fills one: its
// waves hold over 256 registers each), never more than key tiles, and (KV groups x splits) a
// multiple of 8 where possible so that every XCD gets the same number of workgroups.
int splits_for(int H, int G, int max_len) {
  const int ntiles = (max_len + KT - 1) / KT;
  int n = 256 / H;
  if (n < 1) n = 1;
  if (n > ntiles) n = ntiles;
  if (n > MAX_SPLITS) n = MAX_SPLITS;
  for (int m = n; m >= 1 && 2 * m > n; --m)
    if ((G * m) % 8 == 0) return m;
  return n;
}

size_t counter_bytes(int H) { return ((size_t)H * sizeof(unsigned) + 255) & ~(size_t)255; }

template <int HD>
size_t lds_bytes() {
  const size_t vt = (size_t)WAVES * KT * (HD * 2 + 16) + (size_t)EAGLE_MAX_TREE * HD * 4;   // V tiles + cos/sin
  const size_t mg = (size_t)WAVES * 32 * (HD + 4) * 4 + WAVES * 32 * 2 * 4 + 16;
  return vt > mg ? vt : mg;
}

template <int HD>
int launch(const half_t* q, const half_t* k, const half_t* v, long ld, const float* cs, half_t* kc,
           half_t* vc, const uint32_t* bits, const int32_t* len, void* ws, half_t* out, int T, int H,
           int G, long cap, int nsplit, float sl2, hipStream_t st) {
  const size_t lds = lds_bytes<HD>();
  static bool raised = false;           // more than 64 KiB of dynamic LDS has to be requested once
  if (!raised) {
    if (hipFuncSetAttribute((const void*)tree_attn_rope_kernel<HD>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return EAGLE_ERR_HIP;
    raised = true;
  }
  unsigned* counters = static_cast<unsigned*>(ws);
  float* part_ml = reinterpret_cast<float*>(static_cast<unsigned char*>(ws) + counter_bytes(H));
  half_t* part_o = reinterpret_cast<half_t*>(part_ml + (size_t)H * nsplit * 32 * 2);
  const int rep = H / G;
  const int pairs = G * nsplit;
  const int grid = 8 * ((pairs + 7) / 8) * rep;
  hipLaunchKernelGGL(tree_attn_rope_kernel<HD>, dim3(grid), dim3(WAVES * 64), lds, st, q, k, v, ld,
                     cs, kc, vc, bits, len, counters, part_ml, part_o, out, T, H, G, cap, nsplit, sl2);
  return eagle_launch_status();
}

}  // namespace

EAGLE_EXPORT int eagle_rope_table_f32(const int32_t* positions, const float* inv_freqs,
                                      float scaling_factor, int T, int half_dim, float* out,
                                      eagle_stream_t stream) {
  if (!positions || !inv_freqs || !out) return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE || half_dim < 1) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(out)) return EAGLE_ERR_ALIGN;
  const int total = T * half_dim;
  hipLaunchKernelGGL(rope_table_kernel, dim3((total + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), positions, inv_freqs, scaling_factor, out, T,
                     half_dim);
  return eagle_launch_status();
}

EAGLE_EXPORT size_t eagle_tree_attention_rope_workspace_bytes(int H, int hd, int max_len) {
  if (H < 1 || hd < 1 || max_len < 1) return 0;
  return counter_bytes(H) + (size_t)H * MAX_SPLITS * 32 * (2 * sizeof(float) + (size_t)hd * sizeof(half_t));
}

EAGLE_EXPORT int eagle_tree_attention_rope_f16(const void* q_lin, const void* k_lin, const void* v_lin,
                                               long row_stride, const float* rope_cs, void* k_cache,
                                               void* v_cache, const uint32_t* tree_mask_bits,
                                               const int32_t* cache_len_dev, void* out, int T, int H,
                                               int G, int hd, long capacity, int max_len, float scale,
                                               void* workspace, size_t workspace_bytes,
                                               eagle_stream_t stream) {
  if (!q_lin || !k_lin || !v_lin || !rope_cs || !k_cache || !v_cache || !tree_mask_bits ||
      !cache_len_dev || !out)
    return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE || H < 1 || G < 1 || (H % G) != 0 || (hd != 64 && hd != 128) ||
      max_len < T || max_len > capacity || row_stride < hd || (row_stride % 8) != 0)
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q_lin) || !eagle_aligned16(k_lin) || !eagle_aligned16(v_lin) ||
      !eagle_aligned16(rope_cs) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) ||
      !eagle_aligned16(out))
    return EAGLE_ERR_ALIGN;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_tree_attention_rope_workspace_bytes(H, hd, max_len))
    return EAGLE_ERR_WORKSPACE;
  const int nsplit = splits_for(H, G, max_len);
  const float sl2 = scale * 1.4426950408889634f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (hd == 128)
    return launch<128>((const half_t*)q_lin, (const half_t*)k_lin, (const half_t*)v_lin, row_stride,
                       rope_cs, (half_t*)k_cache, (half_t*)v_cache, tree_mask_bits, cache_len_dev,
                       workspace, (half_t*)out, T, H, G, capacity, nsplit, sl2, st);
  return launch<64>((const half_t*)q_lin, (const half_t*)k_lin, (const half_t*)v_lin, row_stride,
                    rope_cs, (half_t*)k_cache, (half_t*)v_cache, tree_mask_bits, cache_len_dev,
                    workspace, (half_t*)out, T, H, G, capacity, nsplit, sl2, st);
}
