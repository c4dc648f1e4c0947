// Integer side of the tree step (gfx950): draft-tree layout, root-to-leaf paths, greedy
// longest-accepted-path selection, KV compaction.  Every kernel here is tiny exact
// integer work; they exist so that a verify step needs no device-to-host round trip.
#include "common.h"

#include <math.h>

namespace {

constexpr int MAXT = EAGLE_MAX_TREE_SLOTS;   // 64: tree tokens the kernels of this file lay out
constexpr int MAXC = 1024;             // draft candidates (k + k*k*depth)

// mlx_eagle.py:217-250 (with topk :24-58 and search_sorted :61-93).
__global__ __launch_bounds__(256) void process_draft_tree_kernel(
    const half_t* __restrict__ scores, const int32_t* __restrict__ tokens,
    const uint32_t* __restrict__ parents_list, const int32_t* __restrict__ sampled,
    int C, int k, int total, int32_t* __restrict__ pos_ids, int32_t* __restrict__ mask_index,
    int32_t* __restrict__ draft_tokens, uint32_t* __restrict__ bits_out) {
  __shared__ float sc[MAXC];
  __shared__ unsigned char picked[MAXC];
  __shared__ int sel[MAXT];
  __shared__ int midx[MAXT];
  __shared__ unsigned long long bits[MAXT];
  const int tid = threadIdx.x;
  // a NaN score ranks as -inf: with the index tie rule the order below is then total, so
  // exactly `total` candidates are picked whatever the scores hold
  for (int i = tid; i < C; i += blockDim.x) {
    const float v = (float)scores[i];
    sc[i] = v != v ? -INFINITY : v;
  }
  __syncthreads();
  // rank in the stable descending order: candidates ahead of i are those with a larger
  // score, or an equal score and a lower flat index
  for (int i = tid; i < C; i += blockDim.x) {
    const float si = sc[i];
    int rank = 0;
    for (int j = 0; j < C; ++j) {
      const float sj = sc[j];
      rank += (sj > si) || (sj == si && j < i);
    }
    picked[i] = rank < total;
  }
  __syncthreads();
  // the picked candidates in ascending flat index
  for (int i = tid; i < C; i += blockDim.x) {
    if (!picked[i]) continue;
    int before = 0;
    for (int j = 0; j < i; ++j) before += picked[j];
    if (before < total) sel[before] = i;
  }
  __syncthreads();
  if (tid < total) {
    const int c = sel[tid];
    draft_tokens[tid + 1] = tokens[c];
    const uint32_t dp = parents_list[c / k];
    // fixed-step left binary search for the flat id dp - 1 (uint32 arithmetic, wraps for dp == 0)
    const uint32_t target = dp - 1u;
    uint32_t low = 0, high = (uint32_t)total;
    int steps = 0;
    while ((1 << steps) < total) ++steps;   // ceil(log2(total))
    for (int s = 0; s < steps; ++s) {
      const uint32_t mid = (low + high) >> 1;
      if (mid < (uint32_t)total) {
        const uint32_t val = (uint32_t)sel[mid];
        if (val < target) low = mid + 1; else high = mid;
      }
    }
    const int mi = (dp == 0u) ? 0 : (int)low + 1;
    midx[tid] = mi;
    mask_index[tid] = mi;
  }
  if (tid == 0) draft_tokens[0] = sampled[0];
  __syncthreads();
  if (tid == 0) {
    // identity rows first, then the sequential OR of mlx_eagle.py:239-243 (a parent slot ahead
    // of its child, which only poisoned scores can produce, then reads an identity row, as the
    // reference's loop over an identity matrix does)
    for (int i = 0; i <= total; ++i) bits[i] = 1ull << i;
    for (int i = 0; i < total; ++i) {
      const int par = midx[i] < 0 ? 0 : (midx[i] > total ? total : midx[i]);
      bits[i + 1] |= bits[par];
    }
  }
  __syncthreads();
  if (tid <= total) {
    // one mask word per row for trees of at most 32 tokens, two (low, high) above that
    if (total + 1 <= 32) {
      bits_out[tid] = (uint32_t)bits[tid];
    } else {
      bits_out[2 * tid] = (uint32_t)bits[tid];
      bits_out[2 * tid + 1] = (uint32_t)(bits[tid] >> 32);
    }
    pos_ids[tid] = __popcll(bits[tid]) - 1;
  }
}

// mlx_eagle.py:254-295.  retrieve [64][64], shape {leaf_num, max_depth + 1}.
__global__ __launch_bounds__(128) void post_process_kernel(const int32_t* __restrict__ pos_ids,
                                                          const int32_t* __restrict__ mask_index,
                                                          int total, int32_t* __restrict__ retrieve,
                                                          int32_t* __restrict__ shape) {
  __shared__ int inner[MAXT + 1];
  __shared__ int depth[MAXT];
  __shared__ int par[MAXT];
  const int tid = threadIdx.x;
  const int T = total + 1;
  if (tid <= MAXT) inner[tid] = 0;
  for (int i = tid; i < MAXT * MAXT; i += blockDim.x) retrieve[i] = -1;
  if (tid < T) depth[tid] = pos_ids[tid];
  if (tid < total) par[tid] = mask_index[tid];
  __syncthreads();
  if (tid < total) {
    const int p = par[tid];
    if (p >= 0 && p <= MAXT) inner[p] = 1;   // benign race: all writers store 1
  }
  __syncthreads();
  if (tid < T && !inner[tid]) {
    int r = 0;
    for (int j = 0; j < tid; ++j) r += !inner[j];
    int cur = tid;
    for (int col = depth[tid]; col >= 0; --col) {
      if (col < MAXT) retrieve[r * MAXT + col] = cur;
      cur = (cur == 0) ? par[total - 1] : par[cur - 1];
      cur = cur < 0 ? 0 : (cur > total ? total : cur);
    }
  }
  if (tid == 0) {
    int n_inner = 0, md = 0;
    for (int j = 0; j <= MAXT; ++j) n_inner += inner[j];
    for (int j = 0; j < T; ++j) md = depth[j] > md ? depth[j] : md;
    shape[0] = total - (n_inner - 1);
    shape[1] = md + 1;
  }
}

// mlx_eagle.py:311-326 on per-node argmax tokens, with the gathers of :582-589.
__global__ __launch_bounds__(128) void greedy_accept_kernel(
    const int32_t* __restrict__ node_argmax, const int32_t* __restrict__ draft_tokens,
    const int32_t* __restrict__ retrieve, const int32_t* __restrict__ shape, int T,
    int32_t* __restrict__ result, int32_t* __restrict__ accepted_tokens) {
  __shared__ int len[MAXT];
  const int tid = threadIdx.x;
  int leaves = shape[0], cols = shape[1];
  leaves = leaves < 1 ? 1 : (leaves > MAXT ? MAXT : leaves);
  cols = cols < 1 ? 1 : (cols > MAXT ? MAXT : cols);
  if (tid < MAXT) len[tid] = -1;
  __syncthreads();
  if (tid < leaves) {
    int n = 0;
    for (int j = 0; j + 1 < cols; ++j) {
      int a = retrieve[tid * MAXT + j];
      int b = retrieve[tid * MAXT + j + 1];
      a = a < 0 ? a + T : a;   // a negative gather index counts from the end
      b = b < 0 ? b + T : b;
      if (draft_tokens[b] == node_argmax[a]) ++n; else break;
    }
    len[tid] = n;
  }
  __syncthreads();
  if (tid == 0) {
    int best = 0, al = len[0];
    for (int r = 1; r < leaves; ++r)
      if (len[r] > al) { al = len[r]; best = r; }
    if (al == 0) best = 0;
    int bonus = retrieve[best * MAXT + al];
    bonus = bonus < 0 ? bonus + T : bonus;
    result[0] = best;
    result[1] = al;
    result[2] = bonus;
    result[3] = node_argmax[bonus];
    for (int j = 0; j < MAXT; ++j) {
      int idx = 0, tok = 0;
      if (j < al) {
        idx = retrieve[best * MAXT + 1 + j];
        const int w = idx < 0 ? idx + T : idx;
        tok = draft_tokens[w];
      }
      result[4 + j] = idx;
      accepted_tokens[j] = tok;
    }
  }
}

// mlx_eagle.py:366-374: rows P + idx[j] -> P + 1 + j, gather first, then scatter.
// grid (G, n_caches); the accepted rows of one head are staged in LDS.
__global__ __launch_bounds__(256) void kv_compact_kernel(half_t* const* __restrict__ caches,
                                                         const int32_t* __restrict__ accept,
                                                         const int32_t* __restrict__ len_dev,
                                                         int hd, long cap) {
  extern __shared__ __attribute__((aligned(16))) unsigned char stage[];
  const int al = accept[1];
  if (al <= 0) return;
  const int n = al > MAXT ? MAXT : al;
  const long P = *len_dev;
  half_t* base = caches[blockIdx.y] + (long)blockIdx.x * cap * hd;
  const int vec_row = hd / 8;
  for (int v = threadIdx.x; v < n * vec_row; v += blockDim.x) {
    const int j = v / vec_row;
    const int c = v % vec_row;
    long src = P + accept[4 + j];
    src = src < 0 ? 0 : (src >= cap ? cap - 1 : src);
    reinterpret_cast<half8_t*>(stage)[v] = *reinterpret_cast<const half8_t*>(base + src * hd + c * 8);
  }
  __syncthreads();
  for (int v = threadIdx.x; v < n * vec_row; v += blockDim.x) {
    const int j = v / vec_row;
    const int c = v % vec_row;
    const long dst = P + 1 + j;
    if (dst < cap)
      *reinterpret_cast<half8_t*>(base + dst * hd + c * 8) = reinterpret_cast<const half8_t*>(stage)[v];
  }
}

// the length saturates at the capacity: a caller that replays steps beyond it gets a full
// cache (the append kernels skip rows at or beyond the capacity), never a length that points
// outside the buffers
__global__ void set_len_after_accept(const int32_t* __restrict__ accept, int32_t* len_dev, long cap) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    const int al = accept[1] < 0 ? 0 : accept[1];
    const long n = (long)*len_dev + al + 1;
    *len_dev = (int32_t)(n < cap ? n : cap);
  }
}

__global__ void fill_i32_kernel(int32_t* dst, int32_t value, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

__global__ void tree_positions_kernel(const int32_t* __restrict__ pos_ids,
                                      const int32_t* __restrict__ len_dev,
                                      int32_t* __restrict__ positions, int T) {
  const int i = threadIdx.x;
  if (i < T) positions[i] = *len_dev + pos_ids[i];
}

__global__ void advance_len_kernel(int32_t* len_dev, int delta) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *len_dev += delta;
}

}  // namespace

EAGLE_EXPORT int eagle_process_draft_tree(const void* scores, const int32_t* tokens,
                                          const uint32_t* parents_list,
                                          const int32_t* sampled_token_dev, int C, int k,
                                          int total, int32_t* tree_position_ids,
                                          int32_t* mask_index, int32_t* draft_tokens,
                                          uint32_t* tree_mask_bits, eagle_stream_t stream) {
  if (!scores || !tokens || !parents_list || !sampled_token_dev || !tree_position_ids ||
      !mask_index || !draft_tokens || !tree_mask_bits)
    return EAGLE_ERR_NULL;
  if (k < 1 || C < 1 || C > MAXC || (C % k) != 0 || total < 1 || total >= MAXT || total > C)
    return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(process_draft_tree_kernel, dim3(1), dim3(256), 0,
                     static_cast<hipStream_t>(stream), (const half_t*)scores, tokens, parents_list,
                     sampled_token_dev, C, k, total, tree_position_ids, mask_index, draft_tokens,
                     tree_mask_bits);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_post_process_draft_tree(const int32_t* tree_position_ids,
                                               const int32_t* mask_index, int total,
                                               int32_t* retrieve_indices, int32_t* shape_out,
                                               eagle_stream_t stream) {
  if (!tree_position_ids || !mask_index || !retrieve_indices || !shape_out) return EAGLE_ERR_NULL;
  if (total < 1 || total >= MAXT) return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(post_process_kernel, dim3(1), dim3(128), 0, static_cast<hipStream_t>(stream),
                     tree_position_ids, mask_index, total, retrieve_indices, shape_out);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_greedy_accept(const int32_t* node_argmax, const int32_t* draft_tokens,
                                     const int32_t* retrieve_indices, const int32_t* shape, int T,
                                     int32_t* result, int32_t* accepted_tokens,
                                     eagle_stream_t stream) {
  if (!node_argmax || !draft_tokens || !retrieve_indices || !shape || !result || !accepted_tokens)
    return EAGLE_ERR_NULL;
  if (T < 1 || T > MAXT) return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(greedy_accept_kernel, dim3(1), dim3(128), 0, static_cast<hipStream_t>(stream),
                     node_argmax, draft_tokens, retrieve_indices, shape, T, result,
                     accepted_tokens);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_kv_compact_f16(void* const* caches_dev, int n_caches, const int32_t* accept,
                                      int32_t* cache_len_dev, int G, int hd, long capacity,
                                      eagle_stream_t stream) {
  if (!caches_dev || !accept || !cache_len_dev) return EAGLE_ERR_NULL;
  if (n_caches < 1 || n_caches > 65535 || G < 1 || hd < 8 || (hd % 8) != 0 || capacity < 2)
    return EAGLE_ERR_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t lds = (size_t)MAXT * hd * 2;
  hipLaunchKernelGGL(kv_compact_kernel, dim3(G, n_caches), dim3(256), lds, st,
                     reinterpret_cast<half_t* const*>(caches_dev), accept, cache_len_dev, hd,
                     capacity);
  hipLaunchKernelGGL(set_len_after_accept, dim3(1), dim3(64), 0, st, accept, cache_len_dev, capacity);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_fill_i32(int32_t* dst, int32_t value, long n, eagle_stream_t stream) {
  if (!dst) return EAGLE_ERR_NULL;
  if (n < 1) return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), dst, value, n);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_tree_positions(const int32_t* tree_position_ids,
                                      const int32_t* cache_len_dev, int32_t* positions, int T,
                                      eagle_stream_t stream) {
  if (!tree_position_ids || !cache_len_dev || !positions) return EAGLE_ERR_NULL;
  if (T < 1 || T > MAXT) return EAGLE_ERR_SHAPE;
  hipLaunchKernelGGL(tree_positions_kernel, dim3(1), dim3(64), 0,
                     static_cast<hipStream_t>(stream), tree_position_ids, cache_len_dev, positions,
                     T);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_advance_len(int32_t* cache_len_dev, int delta, eagle_stream_t stream) {
  if (!cache_len_dev) return EAGLE_ERR_NULL;
  hipLaunchKernelGGL(advance_len_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     cache_len_dev, delta);
  return eagle_launch_status();
}

EAGLE_EXPORT const char* eagle_status_string(int status) {
  switch (status) {
    case EAGLE_OK: return "ok";
    case EAGLE_ERR_NULL: return "required pointer is NULL";
    case EAGLE_ERR_SHAPE: return "dimension outside the supported range";
    case EAGLE_ERR_ALIGN: return "pointer is not sufficiently aligned";
    case EAGLE_ERR_UNSUPPORTED: return "only group_size=64, bits=4 is supported";
    case EAGLE_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case EAGLE_ERR_HIP: return "HIP runtime error at launch";
    case EAGLE_ERR_ARCH: return "device is not gfx950";
    default: return "unknown status";
  }
}

EAGLE_EXPORT int eagle_abi_version(void) { return 1; }

EAGLE_EXPORT int eagle_check_device(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return EAGLE_ERR_HIP;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return EAGLE_ERR_HIP;
  const char* a = prop.gcnArchName;
  return (a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0')
             ? EAGLE_OK
             : EAGLE_ERR_ARCH;
}
