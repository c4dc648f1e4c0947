// Tree-masked grouped-query attention of T <= 32 tree tokens against a KV cache (gfx950).
//
//   out[t, h*hd + d] = sum_j softmax_j( scale * q[h,t,:] . k[g,j,:] + mask[t,j] ) v[g,j,d]
//
// The first P = *cache_len_dev cache rows are the prefix, visible to every tree token;
// rows P .. P+T-1 are the tree tokens, token j visible to token i iff bit j of
// tree_mask_bits[i] is set (the ancestor-or-self mask of mlx_eagle.py:239-248,337-338).
// Call site replaced: mlx_llama.py:185-195.
//
// Split-KV: grid (kv head g, key split s); one wave per query head of the group, so a
// K/V tile is read from memory once per group and shared through LDS.  Per 32-key tile a
// wave computes S^T = K Q^T with v_mfma_f32_32x32x16_f16 (rows = keys, columns = the 32
// tree tokens), runs the online softmax on its accumulator (a lane owns one tree token,
// its partner lane+32 the other half of the keys), and feeds exp(S^T) straight back as
// the B operand of O^T += V^T P^T; only V needs a transposed (16-bit) read from LDS.
// Partial (m, l, O) per split go to a workspace and a second kernel merges them.
#include "common.h"

#include <math.h>

namespace {

constexpr int KT = 32;   // keys per tile

template <int HD>
__global__ __launch_bounds__(512) void tree_attn_split_kernel(
    const half_t* __restrict__ q, const half_t* __restrict__ kc, const half_t* __restrict__ vc,
    const uint32_t* __restrict__ mask_bits, const int32_t* __restrict__ len_dev,
    float* __restrict__ part_o, float* __restrict__ part_ml, int T, int H, int G, long cap,
    int tiles_per_split, float scale_log2e) {
  constexpr int KSTEPS = HD / 16;       // MFMA steps over the head dimension for S
  constexpr int DB = HD / 32;           // 32-wide blocks of the head dimension for O
  constexpr int STR = HD * 2 + 16;      // LDS row stride in bytes (pad: conflict-free reads)
  constexpr int VEC_ROW = HD / 8;       // 16-byte vectors per K/V row
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  unsigned char* ldsK = lds;
  unsigned char* ldsV = lds + KT * STR;

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

  const int P = *len_dev;
  const int Ltot = P + T;
  const int ntiles = (Ltot + KT - 1) / KT;
  const int t0 = split * tiles_per_split;
  const int t1 = min(t0 + tiles_per_split, ntiles);

  half8_t qreg[KSTEPS];
#pragma unroll
  for (int kk = 0; kk < KSTEPS; ++kk) {
    qreg[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (ql < T)
      qreg[kk] = *reinterpret_cast<const half8_t*>(q + ((long)head * T + ql) * HD + kk * 16 + hb * 8);
  }
  const uint32_t mybits = ql < T ? mask_bits[ql] : 0u;

  float m_run = -INFINITY, l_run = 0.f;
  float16_t o_acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[db][i] = 0.f;

  const half_t* kbase_ptr = kc + (long)g * cap * HD;
  const half_t* vbase_ptr = vc + (long)g * cap * HD;

  for (int tile = t0; tile < t1; ++tile) {
    const int kb = tile * KT;
    __syncthreads();   // every wave is done with the previous tile
    for (int v = tid; v < KT * VEC_ROW; v += nthr) {
      const int row = v / VEC_ROW;
      const int c = v % VEC_ROW;
      const int kidx = kb + row;
      half8_t kv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      half8_t vv = kv;
      if (kidx < Ltot) {
        kv = *reinterpret_cast<const half8_t*>(kbase_ptr + (long)kidx * HD + c * 8);
        vv = *reinterpret_cast<const half8_t*>(vbase_ptr + (long)kidx * HD + c * 8);
      }
      *reinterpret_cast<half8_t*>(ldsK + row * STR + c * 16) = kv;
      *reinterpret_cast<half8_t*>(ldsV + row * STR + c * 16) = vv;
    }
    __syncthreads();

    // S^T[key][token] = sum_d K[key][d] Q[token][d]
    float16_t sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      const half8_t a = *reinterpret_cast<const half8_t*>(ldsK + ql * STR + kk * 32 + hb * 16);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[kk], sacc, 0, 0, 0);
    }

    // accumulator register i of this lane is key 8*(i/4) + 4*hb + i%4 of the tile
    float sv[16];
    float bm = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb + 8 * (i >> 2) + 4 * hb + (i & 3);
      const int rel = key - P;
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
  }

  // partials: part_ml [H][nsplit][32][2], part_o [H][nsplit][32][HD]
  const long slot = ((long)head * nsplit + split) * 32 + ql;
  if (hb == 0) {
    part_ml[slot * 2 + 0] = m_run;
    part_ml[slot * 2 + 1] = l_run;
  }
  float* po = part_o + slot * HD;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int d0 = db * 32 + 8 * i4 + 4 * hb;
      float4_t v = float4_t{o_acc[db][4 * i4 + 0], o_acc[db][4 * i4 + 1], o_acc[db][4 * i4 + 2],
                            o_acc[db][4 * i4 + 3]};
      *reinterpret_cast<float4_t*>(po + d0) = v;
    }
}

// Merge the splits: grid (T, H), HD/2 threads... one thread per two output elements.
template <int HD>
__global__ void tree_attn_merge_kernel(const float* __restrict__ part_o,
                                       const float* __restrict__ part_ml,
                                       half_t* __restrict__ out, int T, int H, int nsplit) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;
  const int d = threadIdx.x * 2;
  float mx = -INFINITY;
  for (int s = 0; s < nsplit; ++s)
    mx = fmaxf(mx, part_ml[(((long)head * nsplit + s) * 32 + t) * 2]);
  float den = 0.f, a0 = 0.f, a1 = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const long slot = ((long)head * nsplit + s) * 32 + t;
    const float m = part_ml[slot * 2];
    if (m == -INFINITY) continue;
    const float wgt = exp2f(m - mx);
    den += wgt * part_ml[slot * 2 + 1];
    a0 += wgt * part_o[slot * HD + d];
    a1 += wgt * part_o[slot * HD + d + 1];
  }
  half2_t o = half2_t{(half_t)(a0 / den), (half_t)(a1 / den)};
  *reinterpret_cast<half2_t*>(out + ((long)t * H + head) * HD + d) = o;
}

int tiles_per_split_for(int max_len, int G) {
  const int ntiles = (max_len + KT - 1) / KT;
  int want_splits = 256 / (G > 0 ? G : 1);   // about one workgroup per compute unit
  if (want_splits < 1) want_splits = 1;
  int tps = (ntiles + want_splits - 1) / want_splits;
  if (tps < 4) tps = 4;                      // keep the partial traffic below the KV traffic
  return tps;
}

}  // namespace

EAGLE_EXPORT size_t eagle_tree_attention_workspace_bytes(int H, int hd, int max_len) {
  if (H < 1 || hd < 1 || max_len < 1) return 0;
  // worst case split count: tiles_per_split >= 4
  const int ntiles = (max_len + KT - 1) / KT;
  const int nsplit = (ntiles + 3) / 4;
  return (size_t)H * nsplit * 32 * (hd + 2) * sizeof(float);
}

EAGLE_EXPORT int eagle_tree_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                                          const uint32_t* tree_mask_bits,
                                          const int32_t* cache_len_dev, void* out, int T, int H,
                                          int G, int hd, long capacity, int max_len, float scale,
                                          void* workspace, size_t workspace_bytes,
                                          eagle_stream_t stream) {
  if (!q || !k_cache || !v_cache || !tree_mask_bits || !cache_len_dev || !out) return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE || H < 1 || G < 1 || (H % G) != 0 || (H / G) > 8 ||
      (hd != 64 && hd != 128) || max_len < T || max_len > capacity)
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) ||
      !eagle_aligned16(out))
    return EAGLE_ERR_ALIGN;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_tree_attention_workspace_bytes(H, hd, max_len))
    return EAGLE_ERR_WORKSPACE;
  const int tps = tiles_per_split_for(max_len, G);
  const int ntiles = (max_len + KT - 1) / KT;
  const int nsplit = (ntiles + tps - 1) / tps;
  float* part_ml = static_cast<float*>(workspace);
  float* part_o = part_ml + (size_t)H * nsplit * 32 * 2;
  const float sl2 = scale * 1.4426950408889634f;
  const int rep = H / G;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t lds = 2 * KT * (hd * 2 + 16);
  if (hd == 128) {
    hipLaunchKernelGGL(tree_attn_split_kernel<128>, dim3(G, nsplit), dim3(rep * 64), lds, st,
                       (const half_t*)q, (const half_t*)k_cache, (const half_t*)v_cache,
                       tree_mask_bits, cache_len_dev, part_o, part_ml, T, H, G, capacity, tps, sl2);
    hipLaunchKernelGGL(tree_attn_merge_kernel<128>, dim3(T, H), dim3(64), 0, st, part_o, part_ml,
                       (half_t*)out, T, H, nsplit);
  } else {
    hipLaunchKernelGGL(tree_attn_split_kernel<64>, dim3(G, nsplit), dim3(rep * 64), lds, st,
                       (const half_t*)q, (const half_t*)k_cache, (const half_t*)v_cache,
                       tree_mask_bits, cache_len_dev, part_o, part_ml, T, H, G, capacity, tps, sl2);
    hipLaunchKernelGGL(tree_attn_merge_kernel<64>, dim3(T, H), dim3(32), 0, st, part_o, part_ml,
                       (half_t*)out, T, H, nsplit);
  }
  return eagle_launch_status();
}
