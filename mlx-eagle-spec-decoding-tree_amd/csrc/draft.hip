// Draft-side tree expansion (gfx950): log-softmax + top-k of the draft logits and the
// per-level bookkeeping of generate_draft_tree (mlx_eagle.py:97-213, 410-412), kept on the
// device so that the expansion loop needs no device-to-host round trip.
//
// Scores are carried in fp16, as the reference carries them in the model dtype; every
// ordering is "larger score first, equal scores lowest index first".
#include "common.h"

#include <math.h>

namespace {

constexpr int TOPK_MAX = 8;          // k of the expansion (candidates per node)
constexpr int CHUNK = 4096;          // logits per workgroup
constexpr int THREADS = 256;

struct Cand {
  float v;
  int i;
};
__device__ inline Cand better(Cand a, Cand b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}
__device__ inline Cand wave_best(Cand a) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Cand b;
    b.v = __shfl_xor(a.v, o, 64);
    b.i = __shfl_xor(a.i, o, 64);
    a = better(a, b);
  }
  return a;
}

// Best candidate of the block; every thread gets it.  red: THREADS / 64 entries.
__device__ inline Cand block_best(Cand c, Cand* red) {
  c = wave_best(c);
  __syncthreads();                   // red is free again
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  Cand b = red[0];
#pragma unroll
  for (int w = 1; w < THREADS / 64; ++w) b = better(b, red[w]);
  return b;
}

__device__ inline const half_t* row_ptr(const half_t* logits, const int32_t* row_index, int row,
                                        long V) {
  const long r = row_index ? (long)row_index[row] : (long)row;
  return logits + r * V;
}

// Pass 1: per chunk, the maximum and sum of exp(x - max).  Grid (chunks, rows).
__global__ __launch_bounds__(THREADS) void lse_partial_kernel(
    const half_t* __restrict__ logits, const int32_t* __restrict__ row_index, long V,
    float* __restrict__ pm, float* __restrict__ ps) {
  __shared__ float red[THREADS / 64];
  const int row = blockIdx.y, ch = blockIdx.x, nch = gridDim.x;
  const half_t* r = row_ptr(logits, row_index, row, V);
  const long beg = (long)ch * CHUNK;
  float x[CHUNK / THREADS];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < CHUNK / THREADS; ++j) {
    const long i = beg + threadIdx.x + (long)j * THREADS;
    x[j] = i < V ? (float)r[i] : -INFINITY;
    m = fmaxf(m, x[j]);
  }
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < CHUNK / THREADS; ++j) s += x[j] == -INFINITY ? 0.f : expf(x[j] - m);
  s = wave_sum(s);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    pm[row * nch + ch] = m;
    ps[row * nch + ch] = (red[0] + red[1]) + (red[2] + red[3]);
  }
}

// Row statistics from the partials, the same arithmetic in every workgroup that needs them.
__device__ inline void row_stats(const float* pm, const float* ps, int row, int nch, float* M,
                                 float* S) {
  float m = -INFINITY;
  for (int c = 0; c < nch; ++c) m = fmaxf(m, pm[row * nch + c]);
  float s = 0.f;
  for (int c = 0; c < nch; ++c) {
    const float pmc = pm[row * nch + c];
    if (pmc != -INFINITY) s += ps[row * nch + c] * expf(pmc - m);
  }
  *M = m;
  *S = s;
}

// The fp16 log-probability the reference would hold for logit x.
//   MODE 0 (mlx_eagle.py:410-412): topk over the logits, then fp16(x) - fp16(logsumexp)
//   MODE 1 (mlx_eagle.py:103):     log(softmax(x)) with both tensors materialised in fp16
template <int MODE>
__device__ inline float score_of(float x, float M, float S, float lse16) {
  if (MODE == 0) return (float)(half_t)(x - lse16);
  const float p16 = (float)(half_t)(expf(x - M) / S);
  return (float)(half_t)logf(p16);
}

// Pass 2: per chunk the k best entries by the ordering key (MODE 0: the logit; MODE 1: the
// fp16 log-probability, in which distinct logits can tie).  Grid (chunks, rows).
template <int MODE>
__global__ __launch_bounds__(THREADS) void topk_partial_kernel(
    const half_t* __restrict__ logits, const int32_t* __restrict__ row_index, long V, int k,
    const float* __restrict__ pm, const float* __restrict__ ps, float* __restrict__ pv,
    int32_t* __restrict__ pi) {
  __shared__ Cand red[THREADS / 64];
  const int row = blockIdx.y, ch = blockIdx.x, nch = gridDim.x;
  const half_t* r = row_ptr(logits, row_index, row, V);
  float M = 0.f, S = 1.f;
  if (MODE == 1) row_stats(pm, ps, row, nch, &M, &S);
  const long beg = (long)ch * CHUNK;
  float key[CHUNK / THREADS];
#pragma unroll
  for (int j = 0; j < CHUNK / THREADS; ++j) {
    const long i = beg + threadIdx.x + (long)j * THREADS;
    key[j] = -INFINITY;
    if (i < V) key[j] = MODE == 0 ? (float)r[i] : score_of<1>((float)r[i], M, S, 0.f);
  }
  unsigned taken = 0;                 // bit j: key[j] has been handed out
  for (int n = 0; n < k; ++n) {
    Cand c{-INFINITY, 0x7fffffff};
#pragma unroll
    for (int j = 0; j < CHUNK / THREADS; ++j) {
      const long i = beg + threadIdx.x + (long)j * THREADS;
      if (!((taken >> j) & 1u) && i < V) c = better(c, Cand{key[j], (int)i});
    }
    const Cand b = block_best(c, red);
#pragma unroll
    for (int j = 0; j < CHUNK / THREADS; ++j)
      if ((int)(beg + threadIdx.x + (long)j * THREADS) == b.i) taken |= 1u << j;
    if (threadIdx.x == 0) {
      pv[((long)row * nch + ch) * TOPK_MAX + n] = b.v;
      pi[((long)row * nch + ch) * TOPK_MAX + n] = b.i;     // 0x7fffffff: chunk exhausted
    }
  }
}

// Pass 3: one workgroup per row merges the chunk candidates and writes indices and fp16 scores.
template <int MODE>
__global__ __launch_bounds__(THREADS) void topk_merge_kernel(
    const half_t* __restrict__ logits, const int32_t* __restrict__ row_index, long V, int k,
    int nch, const float* __restrict__ pm, const float* __restrict__ ps,
    const float* __restrict__ pv, const int32_t* __restrict__ pi, int32_t* __restrict__ out_index,
    half_t* __restrict__ out_score) {
  __shared__ Cand red[THREADS / 64];
  const int row = blockIdx.x;
  const int ncand = nch * TOPK_MAX;
  float M, S;
  row_stats(pm, ps, row, nch, &M, &S);
  const float lse16 = (float)(half_t)(M + logf(S));
  const half_t* r = row_ptr(logits, row_index, row, V);
  int last = -1;
  float last_v = INFINITY;
  for (int n = 0; n < k; ++n) {
    // best candidate that comes after the previous pick in the ordering
    Cand c{-INFINITY, 0x7fffffff};
    for (int j = threadIdx.x; j < ncand; j += THREADS) {
      const int slot = j % TOPK_MAX;
      if (slot >= k) continue;
      const Cand e{pv[(long)row * ncand + j], pi[(long)row * ncand + j]};
      if (e.i == 0x7fffffff) continue;
      const bool after = e.v < last_v || (e.v == last_v && e.i > last);
      if (after) c = better(c, e);
    }
    const Cand b = block_best(c, red);
    last = b.i;
    last_v = b.v;
    if (threadIdx.x == 0) {
      const int idx = b.i == 0x7fffffff ? 0 : b.i;
      out_index[row * k + n] = idx;
      out_score[row * k + n] = MODE == 0 ? (half_t)score_of<0>((float)r[idx], M, S, lse16) : (half_t)b.v;
    }
  }
}

// mlx_eagle.py:130-141: state before the first expansion level.
//   saved_scores / saved_tokens [k + k*k*depth], parents [1 + k*depth], mask_words [k][2],
//   cur_scores [k] fp16, cur_ids [k].
__global__ void draft_tree_init_kernel(const int32_t* __restrict__ topk_index,
                                       const half_t* __restrict__ topk_score, int k,
                                       half_t* __restrict__ saved_scores,
                                       int32_t* __restrict__ saved_tokens,
                                       uint32_t* __restrict__ parents, half_t* __restrict__ cur_scores,
                                       int32_t* __restrict__ cur_ids, uint32_t* __restrict__ mask_words) {
  const int r = threadIdx.x;
  if (r == 0) parents[0] = 0u;
  if (r < k) {
    saved_scores[r] = topk_score[r];
    saved_tokens[r] = topk_index[r];
    parents[1 + r] = (uint32_t)r + 1u;      // level 0: arange(k) + 1 (mlx_eagle.py:155-162)
    cur_scores[r] = topk_score[r];
    cur_ids[r] = topk_index[r];
    mask_words[2 * r] = 1u << r;            // the identity block of level 0 (mlx_eagle.py:171)
    mask_words[2 * r + 1] = 0u;
  }
}

// process_generate_tree_iteration (mlx_eagle.py:97-115) after the per-row top-k, plus what
// generate_draft_tree does with its results (mlx_eagle.py:157-162, 171, 194-207).  One wave;
// lane c is candidate c = k * row + column of the level's k x k table.
__global__ __launch_bounds__(64) void draft_tree_level_kernel(
    const int32_t* __restrict__ topk_index, const half_t* __restrict__ topk_score, int level, int k,
    int depth, half_t* __restrict__ saved_scores, int32_t* __restrict__ saved_tokens,
    uint32_t* __restrict__ parents, half_t* __restrict__ cur_scores, int32_t* __restrict__ cur_ids,
    uint32_t* __restrict__ mask_words, int32_t* __restrict__ out_ids,
    int32_t* __restrict__ topk_cs_index) {
  __shared__ float cu[64];
  __shared__ uint32_t old_mask[2 * TOPK_MAX];
  const int c = threadIdx.x;
  const int kk = k * k;
  float mine = -INFINITY;
  int tok = 0;
  if (c < kk) {
    // cumulative score in fp16 (mlx_eagle.py:106)
    mine = (float)(half_t)((float)topk_score[c] + (float)cur_scores[c / k]);
    tok = topk_index[c];
    saved_scores[k + kk * level + c] = (half_t)mine;
    saved_tokens[k + kk * level + c] = tok;
  }
  cu[c] = mine;
  if (c < 2 * k) old_mask[c] = mask_words[c];
  __syncthreads();
  int rank = 0;
  for (int j = 0; j < kk; ++j) rank += (cu[j] > mine) || (cu[j] == mine && j < c);
  if (c < kk && rank < k) {
    const int parent_row = c / k;
    topk_cs_index[rank] = c;
    out_ids[rank] = parent_row;
    cur_scores[rank] = (half_t)mine;
    cur_ids[rank] = tok;
    if (level + 1 < depth) {
      // rows of the next level's block of the parents table: selected flat id + 1
      const uint32_t bias = 1u + (uint32_t)kk * (uint32_t)level + (uint32_t)k;
      parents[1 + k * (level + 1) + rank] = (uint32_t)c + bias;
    }
    // children inherit the parent's row (mlx_eagle.py:207) and see themselves in the next
    // identity block (mlx_eagle.py:171)
    const int col = k * (level + 1) + rank;
    uint32_t lo = old_mask[2 * parent_row], hi = old_mask[2 * parent_row + 1];
    if (col < 32) lo |= 1u << col; else if (col < 64) hi |= 1u << (col - 32);
    mask_words[2 * rank] = lo;
    mask_words[2 * rank + 1] = hi;
  }
}

// Loop state of the speculative step kept on the device (mlx_eagle.py:393-394, 591-599).
__global__ void spec_begin_kernel(const int32_t* __restrict__ draft_len,
                                  const int32_t* __restrict__ accept, int32_t* __restrict__ expand_len,
                                  int32_t* __restrict__ write_len) {
  if (threadIdx.x == 0) {
    const int32_t v = *draft_len + 1 + accept[1];     // draft_offset (mlx_eagle.py:394)
    *expand_len = v;
    *write_len = v;
  }
}

__global__ void spec_update_kernel(const int32_t* __restrict__ accept,
                                   const int32_t* __restrict__ accepted_tokens, int32_t* __restrict__ y,
                                   int y_len, int32_t* __restrict__ draft_len,
                                   const int32_t* __restrict__ expand_len, int32_t* __restrict__ root_token,
                                   int32_t* __restrict__ out_tokens, int32_t* __restrict__ out_count,
                                   int max_out) {
  const int j = threadIdx.x;
  const int a = accept[1];
  const int32_t next = accept[3];
  const int base = *out_count;
  int32_t v = 0;
  if (j < a) v = accepted_tokens[j]; else if (j == a) v = next;
  if (j < y_len) y[j] = v;                            // accepted tokens, bonus token, zero padding
  if (j <= a && base + j < max_out) out_tokens[base + j] = v;
  __syncthreads();
  if (j == 0) {
    *draft_len = *expand_len;                         // the expansion rows are dropped (:593-594)
    *root_token = next;
    *out_count = base + a + 1;
  }
}

inline int chunks_for(long V) { return (int)((V + CHUNK - 1) / CHUNK); }

}  // namespace

EAGLE_EXPORT size_t eagle_logsoftmax_topk_workspace_bytes(int R, long V) {
  if (R < 1 || V < 1) return 0;
  const size_t nch = (size_t)chunks_for(V);
  return (size_t)R * nch * (2 + 2 * TOPK_MAX) * sizeof(float);
}

EAGLE_EXPORT int eagle_logsoftmax_topk_f16(const void* logits, const int32_t* row_index, int R, long V,
                                           int k, int mode, int32_t* out_index, void* out_score,
                                           void* workspace, size_t workspace_bytes,
                                           eagle_stream_t stream) {
  if (!logits || !out_index || !out_score) return EAGLE_ERR_NULL;
  if (R < 1 || R > EAGLE_MAX_TREE || V < 1 || k < 1 || k > TOPK_MAX || k > V) return EAGLE_ERR_SHAPE;
  if (mode != 0 && mode != 1) return EAGLE_ERR_UNSUPPORTED;
  if (!workspace || !eagle_aligned16(workspace) ||
      workspace_bytes < eagle_logsoftmax_topk_workspace_bytes(R, V))
    return EAGLE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nch = chunks_for(V);
  float* pm = static_cast<float*>(workspace);
  float* ps = pm + (size_t)R * nch;
  float* pv = ps + (size_t)R * nch;
  int32_t* pi = reinterpret_cast<int32_t*>(pv + (size_t)R * nch * TOPK_MAX);
  const half_t* lg = static_cast<const half_t*>(logits);
  half_t* os = static_cast<half_t*>(out_score);
  hipLaunchKernelGGL(lse_partial_kernel, dim3(nch, R), dim3(THREADS), 0, st, lg, row_index, V, pm, ps);
  if (mode == 0) {
    hipLaunchKernelGGL(topk_partial_kernel<0>, dim3(nch, R), dim3(THREADS), 0, st, lg, row_index, V, k,
                       pm, ps, pv, pi);
    hipLaunchKernelGGL(topk_merge_kernel<0>, dim3(R), dim3(THREADS), 0, st, lg, row_index, V, k, nch, pm,
                       ps, pv, pi, out_index, os);
  } else {
    hipLaunchKernelGGL(topk_partial_kernel<1>, dim3(nch, R), dim3(THREADS), 0, st, lg, row_index, V, k,
                       pm, ps, pv, pi);
    hipLaunchKernelGGL(topk_merge_kernel<1>, dim3(R), dim3(THREADS), 0, st, lg, row_index, V, k, nch, pm,
                       ps, pv, pi, out_index, os);
  }
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_draft_tree_init(const int32_t* topk_index, const void* topk_score, int k,
                                       void* saved_scores, int32_t* saved_tokens, uint32_t* parents,
                                       void* cur_scores, int32_t* cur_ids, uint32_t* mask_words,
                                       eagle_stream_t stream) {
  if (!topk_index || !topk_score || !saved_scores || !saved_tokens || !parents || !cur_scores ||
      !cur_ids || !mask_words)
    return EAGLE_ERR_NULL;
  if (k < 1 || k > TOPK_MAX) return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(draft_tree_init_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     topk_index, static_cast<const half_t*>(topk_score), k,
                     static_cast<half_t*>(saved_scores), saved_tokens, parents,
                     static_cast<half_t*>(cur_scores), cur_ids, mask_words);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_draft_tree_level(const int32_t* topk_index, const void* topk_score, int level,
                                        int k, int depth, void* saved_scores, int32_t* saved_tokens,
                                        uint32_t* parents, void* cur_scores, int32_t* cur_ids,
                                        uint32_t* mask_words, int32_t* out_ids,
                                        int32_t* topk_cs_index, eagle_stream_t stream) {
  if (!topk_index || !topk_score || !saved_scores || !saved_tokens || !parents || !cur_scores ||
      !cur_ids || !mask_words || !out_ids || !topk_cs_index)
    return EAGLE_ERR_NULL;
  if (k < 1 || k > TOPK_MAX || depth < 1 || level < 0 || level >= depth || k * depth > 64)
    return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(draft_tree_level_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     topk_index, static_cast<const half_t*>(topk_score), level, k, depth,
                     static_cast<half_t*>(saved_scores), saved_tokens, parents,
                     static_cast<half_t*>(cur_scores), cur_ids, mask_words, out_ids, topk_cs_index);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_spec_begin(const int32_t* draft_len_dev, const int32_t* accept,
                                  int32_t* expand_len_dev, int32_t* write_len_dev,
                                  eagle_stream_t stream) {
  if (!draft_len_dev || !accept || !expand_len_dev || !write_len_dev) return EAGLE_ERR_NULL;
  hipLaunchKernelGGL(spec_begin_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     draft_len_dev, accept, expand_len_dev, write_len_dev);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_spec_update(const int32_t* accept, const int32_t* accepted_tokens, int32_t* y,
                                   int y_len, int32_t* draft_len_dev, const int32_t* expand_len_dev,
                                   int32_t* root_token_dev, int32_t* out_tokens, int32_t* out_count_dev,
                                   int max_out, eagle_stream_t stream) {
  if (!accept || !accepted_tokens || !y || !draft_len_dev || !expand_len_dev || !root_token_dev ||
      !out_tokens || !out_count_dev)
    return EAGLE_ERR_NULL;
  if (y_len < 1 || y_len > 64 || max_out < 1) return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(spec_update_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), accept,
                     accepted_tokens, y, y_len, draft_len_dev, expand_len_dev, root_token_dev, out_tokens,
                     out_count_dev, max_out);
  return eagle_launch_status();
}
