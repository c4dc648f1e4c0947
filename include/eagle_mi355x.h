/*
 * eagle_mi355x.h - C ABI of the MI355X (gfx950) EAGLE-2 tree-verification kernels.
 *
 * Plain pointers and sizes only.  Every pointer argument named `*_dev` or typed
 * as tensor data is a DEVICE pointer; `stream` is a hipStream_t passed as void*.
 * All entry points are asynchronous and stream ordered, never synchronise,
 * never allocate and never retain pointers.  Half-precision tensors are IEEE
 * binary16.  Return value: 0 on success, an eagle_status code otherwise;
 * argument errors are detected on the host before any device work is issued.
 *
 * Each declaration cites the reference interface it replaces
 * (file:line in 0seba/mlx-eagle-spec-decoding-tree).
 *
 * Two groups.  DEFAULT: what the library's own verification step, draft loop and prompt pass
 * call when nothing is chosen by hand: eagle_qmm_w4g64_f16 (+ _workspace_bytes), eagle_qmm_swiglu_*,
 * eagle_qmm_slab_* (partial sums, SwiGLU, their tiled forms and eagle_qmm_tile_w4g64),
 * eagle_qmv_w4g64_f16 / eagle_qmv_rows_w4g64_f16 (one and two rows), eagle_qmm_small_* and
 * eagle_qkv_rope_small_* (a drafter's passes), eagle_qmm_gemm_* (prompt chunks), every rope, norm,
 * attention, embedding, argmax, tree and loop-state entry point.  ON REQUEST: complete and tested,
 * but picked by a caller only: eagle_qmm_plan / eagle_qmm_w4g64_f16_tuned (a launch shape chosen by
 * hand), eagle_slab_sum_f16 (partial sums written out as a plain product),
 * eagle_qmv_rows_w4g64_f16 at three to eight rows, eagle_qmm_w4g64_f16_noalloc (callers that cannot
 * allocate).  There are no experimental entry points.
 */
#ifndef EAGLE_MI355X_H
#define EAGLE_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* eagle_stream_t; /* hipStream_t */

enum eagle_status {
  EAGLE_OK = 0,
  EAGLE_ERR_NULL = 1,        /* required pointer is NULL */
  EAGLE_ERR_SHAPE = 2,       /* a dimension is out of the supported range */
  EAGLE_ERR_ALIGN = 3,       /* pointer not 16-byte aligned */
  EAGLE_ERR_UNSUPPORTED = 4, /* group_size != 64, bits != 4, or a form the shape does not allow */
  EAGLE_ERR_WORKSPACE = 5,   /* workspace missing or too small */
  EAGLE_ERR_HIP = 6,         /* the HIP runtime reported a launch error */
  EAGLE_ERR_ARCH = 7         /* current device is not gfx950 */
};

#define EAGLE_MAX_TREE 32    /* tree tokens per matmul launch and mask word (root + 31 nodes); larger trees take
                                two mask words and the entry points that say so */
#define EAGLE_MAX_TREE_SLOTS 64 /* tree tokens the tree-layout kernels take (root + 63 nodes; the reference's
                                   default is 39 nodes, mlx_eagle.py:390,510) */
#define EAGLE_MAX_CHUNK 2048 /* rows of one causal pass over a prompt chunk */
#define EAGLE_MAX_M 32       /* rows of x accepted by the quantised matmul */

const char* eagle_status_string(int status);
int eagle_abi_version(void);
/* 0 if the current HIP device is gfx950, EAGLE_ERR_ARCH / EAGLE_ERR_HIP otherwise. */
int eagle_check_device(void);

/* ---------------------------------------------------------------------------
 * 4-bit affine quantised matmul, group size 64 (MLX layout).
 *   out[m,n] = fp16( sum_k x[m,k] * (scales[n,k/64]*q[n,k] + biases[n,k/64]) ) (+ bias[n])
 *   q[n,k] = (wq[n,k/8] >> 4*(k%8)) & 15
 *   x [M,K] fp16 row-major, wq [N,K/8] uint32, scales/biases [N,K/64] fp16,
 *   bias [N] fp16 or NULL (added in fp16 after rounding), out [M,N] fp16.
 * Constraints: 1 <= M <= 32, K % 64 == 0, N % 8 == 0, N * K / 2 < 2^32, group_size == 64,
 * bits == 4.
 * Replaces qmm_kernel.matmul (qmm_kernel.py:84-164) with the body
 * kernels/progression/simd_no_swizzle_cast.metal, the mx.quantized_matmul
 * fallback of the patched layer (mlx_model_fwd_bench.py:65-73) and its bias add
 * (:70-71).
 * `workspace` holds split-K partial sums and arrival counters; its first
 * EAGLE_QMM_COUNTER_BYTES bytes must be zero before the first call (they are
 * left zero by every call).  Calls sharing a workspace must be stream ordered.
 * ------------------------------------------------------------------------- */
#define EAGLE_QMM_COUNTER_BYTES 65536
size_t eagle_qmm_workspace_bytes(int M, int N, int K);
int eagle_qmm_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                        const void* biases, const void* bias, void* out,
                        int M, int N, int K, int group_size, int bits,
                        void* workspace, size_t workspace_bytes, eagle_stream_t stream);
/* The product for a pass of at most 16 rows through a small model (the drafter's passes of the
 * tree loop), with the operators around it folded in, so that a decoder layer needs four of
 * these launches and no norm / add launch (mlx_llama.py:195-196, 214-215, 225-249):
 *   norm_w != NULL: the rows of x are RMS-normalised with norm_w [K] (and eps) before the
 *     product, as eagle_rmsnorm_f16 would (the input / post-attention norm of the layer);
 *   residual != NULL: out = residual + fp16(x . W^T) (the o and down projections; residual may be
 *     `out` itself: h is updated in place);
 *   swiglu != 0: W holds gate and up interleaved in 16-row tiles as for
 *     eagle_qmm_swiglu_w4g64_f16, N = 2 I rows, out [T, I] = silu(g) * u.
 * Otherwise as eagle_qmm_w4g64_f16 (bias [N] or NULL added in fp16 after rounding).  Replaces the
 * launches of eagle_qmm_w4g64_f16 / eagle_qmm_slab_partial_w4g64 and eagle_rmsnorm_f16 /
 * eagle_rmsnorm_slabs_f16 of such a pass.
 * Constraints (eagle_qmm_small_supported): T <= 16; K a multiple of 128, up to 6144 (the waves of
 * a workgroup hold all of x between them); N a multiple of 16 (32 with SwiGLU); every scale
 * below 0.2499 in magnitude (the nibbles are expanded through fp16 subnormals times
 * scale * 2^18); x must not alias out; x, norm_w, wq, residual, out 16-byte aligned. */
int eagle_qmm_small_supported(int T, int N, int K, int norm, int swiglu);
int eagle_qmm_small_w4g64_f16(const void* x, const void* norm_w, float eps, const uint32_t* wq,
                              const void* scales, const void* biases, const void* bias,
                              const void* residual, void* out, int T, int N, int K,
                              int group_size, int bits, int swiglu, eagle_stream_t stream);

/* q|k|v of a small pass with everything around it in one launch: RMSNorm of x (norm_w, or NULL for
 * none), the product with the fused q|k|v matrix [(H + 2 G) hd, D] (+ bias), the rotation of q and
 * k with the per-token (cos, sin) table of eagle_rope_table_f32, and the append of the new K / V
 * rows to the caches at row *cache_len_dev (mlx_llama.py:136-183, 231-233).  Replaces
 * eagle_rmsnorm_f16 + eagle_qmm_w4g64_f16 + eagle_rope_kv_append_table_f16 of such a pass (same
 * formula and roundings as the last of them).
 *   x [T, D] fp16; rope_cs [T, hd / 2, 2] fp32; q_out [H, T, hd] fp16; k_cache, v_cache
 *   [G, capacity, hd] fp16 (rows *cache_len_dev + t are written; rows at or past capacity are not).
 * Constraints (eagle_qkv_rope_small_supported): T <= 16, D a multiple of 128 up to 6144, hd a
 * multiple of 32, scales below 0.2499 in magnitude. */
int eagle_qkv_rope_small_supported(int T, int D, int H, int G, int hd);
int eagle_qkv_rope_small_w4g64_f16(const void* x, const void* norm_w, float eps, const uint32_t* wq,
                                   const void* scales, const void* biases, const void* bias,
                                   const float* rope_cs, void* q_out, void* k_cache, void* v_cache,
                                   const int32_t* cache_len_dev, int T, int D, int H, int G, int hd,
                                   long capacity, int group_size, int bits, eagle_stream_t stream);

/* The product for ONE row of x on the vector ALU (v_dot2_f32_f16 on magic-number fp16 nibbles,
 * sum over the sixteen lanes of a row with DPP), no matrix instructions: the M = 1 case of
 * mx.quantized_matmul (mlx_model_fwd_bench.py:65-73), factorised as in kernels/qmv/1b.metal:121-147.
 * K % 512 == 0 and x plus its group sums must fit LDS (eagle_qmv_supported returns 1); x and wq
 * 16-byte aligned.  out [N] fp16. */
int eagle_qmv_supported(int N, int K);
int eagle_qmv_w4g64_f16(const void* x, const uint32_t* wq, const void* scales, const void* biases,
                        const void* bias, void* out, int N, int K, int group_size, int bits,
                        eagle_stream_t stream);
/* The same for 1..8 rows of x (eagle_qmv_rows_supported): the expanded nibbles of a packed word
 * serve every row, as the reference's batched vector kernel does (kernels/qmv/1b.metal:100-147,
 * qmv.py:226-241); x [M, K], out [M, N].  Measured against the matrix-tile kernel at M = 2, 4, 8
 * by `bench.py --small-m`. */
int eagle_qmv_rows_supported(int M, int N, int K);
int eagle_qmv_rows_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                             const void* biases, const void* bias, void* out, int M, int N, int K,
                             int group_size, int bits, eagle_stream_t stream);

/* The same matmul for callers that cannot allocate or bring a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  The split-K partial sums and arrival counters live in a fixed array of
 * EAGLE_QMM_NOALLOC_SCRATCH_BYTES in device memory that the library owns (one copy per GPU,
 * held until the process ends); the call allocates and frees nothing.  A shape whose workspace
 * (eagle_qmm_workspace_bytes) exceeds that size returns EAGLE_ERR_WORKSPACE.  Same kernels,
 * launch shapes and results, bit for bit, as eagle_qmm_w4g64_f16.  Every call on one GPU
 * shares the array: calls that overlap on one GPU (different streams) race; the counters are
 * cleared at the start of every call. */
#define EAGLE_QMM_NOALLOC_SCRATCH_BYTES (8u << 20)
size_t eagle_qmm_noalloc_scratch_bytes(void);
int eagle_qmm_w4g64_f16_noalloc(const void* x, const uint32_t* wq, const void* scales,
                                const void* biases, const void* bias, void* out,
                                int M, int N, int K, int group_size, int bits,
                                eagle_stream_t stream);
/* The launch shape the library would pick: plan5 = {streaming waves per workgroup,
 * phases (column units each streaming wave owns, one after the other), K slabs, tile
 * ranges (workgroups per slab), columns per unit (256 for M <= 16; 128 or 256 above)}. */
int eagle_qmm_plan(int M, int N, int K, int* plan5);
/* Same matmul with the launch shape forced (tuning sweeps and tests).  nw <= 14 (<= 10
 * with 256-column units at M > 16), phases <= 8, nw * phases * splits must cover K with no
 * empty slab, 1 <= ranges <= ceil(N / 16), unit_cols 0 (the default for M), 128 or 256,
 * and the shape must fit LDS, else EAGLE_ERR_SHAPE. */
size_t eagle_qmm_workspace_bytes_tuned(int M, int N, int splits);
int eagle_qmm_w4g64_f16_tuned(const void* x, const uint32_t* wq, const void* scales,
                              const void* biases, const void* bias, void* out,
                              int M, int N, int K, int nw, int phases, int splits, int ranges,
                              int unit_cols, void* workspace, size_t workspace_bytes, eagle_stream_t stream);

/* SwiGLU form of the same matmul for the MLP gate and up projections (mlx_llama.py:214-215:
 * down(silu(gate(x)) * up(x))).  wq / scales / biases / bias hold both projections with their
 * rows interleaved in 16-row tiles: gate rows 0..15, up rows 0..15, gate rows 16..31, ...
 * (N = 2 * intermediate size, N % 32 == 0).  out [M, N/2] = fp16(fp16(silu(g)) * u) with
 * g, u the fp16 results of the two projections, i.e. the values the separate launches and
 * eagle_silu_mul_f16 produce.  Workspace as for eagle_qmm_w4g64_f16 with the same M, N, K. */
int eagle_qmm_swiglu_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                               const void* biases, const void* bias, void* out,
                               int M, int N, int K, int group_size, int bits,
                               void* workspace, size_t workspace_bytes, eagle_stream_t stream);

/* The same product for any number of rows M, as a tiled MFMA GEMM (128 x 128 output blocks,
 * weights expanded to fp16 in registers): the form for the prompt pass (mlx_eagle.py:522-533,
 * where mlx_model_fwd_bench.py:65-73 falls back to mx.quantized_matmul because the row count is
 * not 8..32).  Bound by the matrix cores, not by the weight stream, from a few hundred rows on.
 * No workspace.  N % 8 == 0, K % 64 == 0; bias (may be NULL) 8-byte aligned. */
int eagle_qmm_gemm_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                             const void* biases, const void* bias, void* out, int M, int N, int K,
                             int group_size, int bits, eagle_stream_t stream);
/* The same with the SwiGLU epilogue of eagle_qmm_swiglu_w4g64_f16 (gate and up rows interleaved
 * in 16-row tiles, N = 2 * intermediate size, N % 32 == 0, out [M, N / 2]): the gate|up projection
 * of a prompt chunk without the intermediate [M, N] tensor and the eagle_silu_mul_f16 launch
 * (mlx_llama.py:214-215). */
int eagle_qmm_gemm_swiglu_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                    const void* biases, const void* bias, void* out, int M, int N,
                                    int K, int group_size, int bits, eagle_stream_t stream);

/* The same product for 1..64 rows in the slab form, with the result left as fp32 partial sums:
 * every workgroup owns 128 weight rows and one K slab of `steps_per_slab` quantisation groups
 * (a multiple of 8), moves x through LDS eight groups at a time and expands the weights to fp16
 * in registers for v_mfma_f32_32x32x16_f16.  partial [slabs][R][N] fp32, R = 32 for M <= 32 and 64
 * for 33..64 rows (a tree above 32 tokens; every expanded weight then feeds two matrix
 * instructions) (rows >= M are not written),
 * slabs = eagle_qmm_slab_count(K, steps_per_slab) (0 for a shape the form does not take:
 * K % 128 == 0 is required; scales and biases 16-byte aligned when K % 512 == 0, 4-byte aligned
 * otherwise).  The product is
 * fp16(sum over the slabs, in slab order) (+ fp16 bias): the kernel that consumes it adds the
 * slabs while it loads (eagle_rmsnorm_slabs_f16, eagle_rope_kv_append_slabs_f16), or
 * eagle_slab_sum_f16 writes it out.  No counters, no workspace.  For the small projections of
 * a verification step this is about twice as fast as a kernel that reduces its own slabs.
 * Replaces the same mx.quantized_matmul call sites (mlx_model_fwd_bench.py:65-73). */
int eagle_qmm_slab_count(int K, int steps_per_slab);
/* K steps per slab recommended for this product, 0 where eagle_qmm_w4g64_f16 is the faster form
 * (few rows, very many weight rows, or K not a multiple of 512). */
int eagle_qmm_slab_steps(int M, int N, int K);
size_t eagle_qmm_slab_partial_bytes(int N, int K, int steps_per_slab);             /* M <= 32 */
size_t eagle_qmm_slab_partial_bytes_rows(int M, int N, int K, int steps_per_slab); /* M <= 64 */
int eagle_qmm_slab_partial_w4g64(const void* x, const uint32_t* wq, const void* scales,
                                 const void* biases, float* partial, size_t partial_bytes,
                                 int M, int N, int K, int group_size, int bits,
                                 int steps_per_slab, eagle_stream_t stream);
/* gate|up + SwiGLU (mlx_llama.py:214-215) for 1..64 rows on the slab kernel with one slab over all
 * of K: operands as eagle_qmm_swiglu_w4g64_f16 (gate and up rows interleaved in 16-row tiles, bias
 * [N] interleaved likewise or NULL), out [M, N/2] fp16 = silu(g) * u with the same roundings.
 * For 33..64 rows (a tree above 32 tokens) one launch in place of two of the 32-row kernel. */
int eagle_qmm_slab_swiglu_supported(int M, int N, int K);
/* 1 where this form measured faster than eagle_qmm_swiglu_w4g64_f16 (always above 32 rows). */
int eagle_qmm_slab_swiglu_preferred(int M, int N, int K);
int eagle_qmm_slab_swiglu_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                    const void* biases, const void* bias, void* out, int M, int N, int K,
                                    int group_size, int bits, eagle_stream_t stream);
/* The weights of a projection in the layout the 32-row slab kernels stream fastest.  The
 * reference keeps every matrix row-major ([N, K/8] words: M = w.shape[0], qmm_kernel.py:99-101)
 * and re-orders the words offline only under its --swizzle option (swizzle.py:41-55, applied at
 * qmm_kernel.py:221-225); read row-major, a wave's load
 * touches 32 cache lines for 1 KB.  eagle_qmm_tile_w4g64 re-lays a matrix out once (not in
 * place) as
 *   wt  [N/32 tiles][K/64 groups][64 lanes][4 words]: lane l of a wave holds words 4 (l / 32) ..
 *       4 (l / 32) + 3 of the group for row 32 tile + l % 32, so a tile's group is one contiguous
 *       1 KB block in the order the lanes use it;
 *   sbt [N/32 tiles][K/512 chunks][64 lanes][8 halves]: lanes 0..31 the scales of their row for
 *       the chunk's eight groups, lanes 32..63 the biases (eagle_qmm_tiled_sb_bytes bytes).
 * N % 32 == 0, K % 512 == 0, all pointers 16-byte aligned.
 * eagle_qmm_slab_partial_tiled_w4g64 / eagle_qmm_slab_swiglu_tiled_w4g64_f16 are
 * eagle_qmm_slab_partial_w4g64 / eagle_qmm_slab_swiglu_w4g64_f16 for 1..64 rows on that copy
 * (same results, same partial-sum layout, same consumers).  small_scales != 0 promises that
 * every |scale| is below 0.0624: the nibbles are then expanded through fp16 subnormals (scale *
 * 2^20 must be a finite fp16; larger scales give inf / NaN, never a finite wrong value).
 * Replace the same call sites (qmm_kernel.py:84-164, mlx_model_fwd_bench.py:65-73; with the
 * SwiGLU epilogue mlx_llama.py:214-215). */
int eagle_qmm_tiled_supported(int M, int N, int K);
size_t eagle_qmm_tiled_sb_bytes(int N, int K);
int eagle_qmm_tile_w4g64(const uint32_t* wq, const void* scales, const void* biases, uint32_t* wt,
                         void* sbt, int N, int K, int group_size, int bits, eagle_stream_t stream);
int eagle_qmm_slab_partial_tiled_w4g64(const void* x, const uint32_t* wt, const void* sbt,
                                       float* partial, size_t partial_bytes, int M, int N, int K,
                                       int steps_per_slab, int small_scales, eagle_stream_t stream);
int eagle_qmm_slab_swiglu_tiled_w4g64_f16(const void* x, const uint32_t* wt, const void* sbt,
                                          const void* bias, void* out, int M, int N, int K,
                                          int small_scales, eagle_stream_t stream);
/* The whole product from the tiled copy, out [M,N] fp16 (+ bias [N] fp16 or NULL, added in fp16
 * after rounding), for up to 32 rows and a matrix of very many rows: the vocabulary projection
 * (mlx_llama.py:309-312: `lm_head`, or the tied embedding's `as_linear`).  One workgroup per compute
 * unit owns 16 or 20 32-row tiles over all of K, so that a compute unit reads x once.  M <= 32,
 * N % 32 == 0, K % 512 == 0; small_scales as above.  Same value as eagle_qmm_w4g64_f16 to the
 * rounding of the fp16 weights (tolerance of the tests, not bit-identical). */
int eagle_qmm_rows_tiled_supported(int M, int N, int K);
int eagle_qmm_rows_tiled_w4g64_f16(const void* x, const uint32_t* wt, const void* sbt, const void* bias,
                                   void* out, int M, int N, int K, int small_scales,
                                   eagle_stream_t stream);
/* out [M,N] fp16 = fp16(sum of the slabs) (+ bias [N] fp16, 16-byte aligned, may be NULL).  M must
 * be the M of the call that wrote the partial sums (the rows per slab, 32 or 64, follow from it). */
int eagle_slab_sum_f16(const float* partial, int slabs, const void* bias, void* out, int M, int N,
                       eagle_stream_t stream);

/* Quantised embedding gather: out[t,:] = fp16(scales*q + biases) of row ids[t].
 * ids [T] int32, out [T,D] fp16, D % 64 == 0.  Replaces the quantised
 * nn.Embedding lookup of mlx_llama.py:273. */
int eagle_embed_w4g64_f16(const int32_t* ids, const uint32_t* wq, const void* scales,
                          const void* biases, void* out, int T, int D, int V,
                          eagle_stream_t stream);

/* ---------------------------------------------------------------------------
 * RoPE with one position per (batch, token), half-split pairing, fp32 math.
 *   x, out [B,H,L,hd] fp16 contiguous; positions [B,L] int32; inv_freqs [hd/2] fp32.
 * Replaces rope_positions (mlx_arrayed_rope_kernel.py:46-152).
 * ------------------------------------------------------------------------- */
int eagle_rope_arrayed_f16(const void* x, const int32_t* positions, const float* inv_freqs,
                           float scaling_factor, void* out, int B, int H, int L, int hd,
                           eagle_stream_t stream);

/* Fused form used inside the decoder layer: takes the token-major projections
 * q_lin [T,H*hd], k_lin [T,G*hd], v_lin [T,G*hd], rotates q and k at
 * positions[t] and writes q_out [H,T,hd] plus rows *cache_len_dev + t of the
 * K/V caches ([G,capacity,hd]).  row_stride = 0: the three inputs are packed as
 * above; row_stride > 0: all three are column blocks of one [T,row_stride] matrix
 * (a fused q|k|v projection) and consecutive tokens are row_stride elements apart.
 * Covers mlx_llama.py:134-161 and the cache append of :178. */
int eagle_rope_kv_append_f16(const void* q_lin, const void* k_lin, const void* v_lin,
                             const int32_t* positions, const float* inv_freqs,
                             float scaling_factor, void* q_out, void* k_cache, void* v_cache,
                             const int32_t* cache_len_dev, int T, int H, int G, int hd,
                             long capacity, long row_stride, eagle_stream_t stream);

/* ---------------------------------------------------------------------------
 * Tree-masked grouped-query attention of T <= 32 tree tokens against the cache.
 *   q [H,T,hd] fp16 (rotated), k_cache/v_cache [G,capacity,hd] fp16 holding
 *   P = *cache_len_dev prefix rows followed by the T tree rows,
 *   tree_mask_bits [T] uint32: bit j of word i set iff tree token j is visible
 *   to tree token i; prefix rows are visible to every token.
 *   out [T,H*hd] fp16 = softmax(scale*q.k + mask) v, laid out for o_proj.
 * hd must be 64 or 128, scale positive (this and the other attention entry points return
 * EAGLE_ERR_SHAPE otherwise).  Replaces scaled_dot_product_attention with the additive
 * tree mask (mlx_llama.py:185-195, mask from mlx_eagle.py:337-338).
 * ------------------------------------------------------------------------- */
/* max_len bounds prefix + tree rows (P + T) for every launch that uses the workspace. */
size_t eagle_tree_attention_workspace_bytes(int H, int hd, int max_len);
int eagle_tree_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                             const uint32_t* tree_mask_bits, const int32_t* cache_len_dev,
                             void* out, int T, int H, int G, int hd, long capacity,
                             int max_len, float scale, void* workspace,
                             size_t workspace_bytes, eagle_stream_t stream);

/* RMSNorm (mlx_llama.py:225-228,240,247,286): out = w * x * rsqrt(mean(x^2)+eps),
 * fp32 math; x, out [T,D] fp16, w [D] fp16.  With `residual` non-NULL the kernel
 * first forms h = fp16(x + residual), stores it to h_out and normalises h
 * (the residual adds of mlx_llama.py:246,248 fused with the following norm). */
int eagle_rmsnorm_f16(const void* x, const void* residual, const void* w, float eps,
                      void* h_out, void* out, int T, int D, eagle_stream_t stream);
/* The same with x held as fp32 partial sums of K slabs (eagle_qmm_slab_partial_w4g64 with
 * N = D): x = fp16(sum of the slabs).  T <= 64, and T must be the M of the call that wrote the
 * partial sums: a slab holds 32 rows for M <= 32 and 64 rows above, and this kernel derives that
 * stride from T (a smaller T over 64-row slabs would read the wrong rows). */
int eagle_rmsnorm_slabs_f16(const float* partial, int slabs, const void* residual, const void* w,
                            float eps, void* h_out, void* out, int T, int D, eagle_stream_t stream);

/* out = fp16( fp16(silu(g)) * u ); g, u are the two halves of gate_up [T,2*I]
 * when `up` is NULL (g = gate_up[:, :I], u = gate_up[:, I:]) or separate [T,I]
 * tensors.  mlx_llama.py:215. */
int eagle_silu_mul_f16(const void* gate, const void* up, void* out, int T, int I,
                       eagle_stream_t stream);

/* out = fp16(a + b), n elements (residual add, mlx_llama.py:246,248). */
int eagle_add_f16(const void* a, const void* b, void* out, long n, eagle_stream_t stream);

/* eagle_rope_kv_append_f16 with the angles taken from a table of eagle_rope_table_f32
 * (below) instead of positions and frequencies: one table per verify step serves every
 * layer, and the per-layer launch no longer evaluates sincos.  Same angles; the rotated
 * values agree with eagle_rope_kv_append_f16 to one fp16 ulp. */
int eagle_rope_kv_append_table_f16(const void* q_lin, const void* k_lin, const void* v_lin,
                                   const float* rope_cs, void* q_out, void* k_cache, void* v_cache,
                                   const int32_t* cache_len_dev, int T, int H, int G, int hd,
                                   long capacity, long row_stride, eagle_stream_t stream);
/* The same with the fused q|k|v projection held as fp32 partial sums of K slabs
 * (eagle_qmm_slab_partial_w4g64 with N = (H + 2G) hd, rows [q heads | k heads | v heads]):
 * every value is fp16(sum of the slabs) + bias (bias [N] fp16, 16-byte aligned, may be NULL)
 * before the rotation.  T <= 64, and T must be the M of the call that wrote the partial sums (the
 * rows per slab, 32 or 64, follow from it). */
int eagle_rope_kv_append_slabs_f16(const float* partial, int slabs, const void* bias,
                                   const float* rope_cs, void* q_out, void* k_cache, void* v_cache,
                                   const int32_t* cache_len_dev, int T, int H, int G, int hd,
                                   long capacity, eagle_stream_t stream);

/* cos/sin table for eagle_rope_kv_append_table_f16: out[t][i] = (cos, sin)(positions[t] *
 * scaling_factor * inv_freqs[i]), fp32 [T, half_dim, 2]; the same angles as
 * eagle_rope_arrayed_f16 (mlx_arrayed_rope_kernel.py:60-123).  The table depends on the tree
 * positions only, so one call serves every layer of a step. */
int eagle_rope_table_f32(const int32_t* positions, const float* inv_freqs, float scaling_factor,
                         int T, int half_dim, float* out, eagle_stream_t stream);
/* Both table forms take up to EAGLE_MAX_CHUNK rows (a prompt chunk); the other tree entry
 * points take at most EAGLE_MAX_TREE. */

/* Attention of the draft-side expansion (mlx_eagle.py:143-178,207 through mlx_llama.py:185-192):
 * T <= 32 query tokens against the P = *cache_len_dev prefix rows (visible to every query) and
 * the Tk <= 64 cache rows P .. P+Tk-1 that follow them, of which query t sees row j iff bit
 * (j % 32) of mask_words[2*t + j/32] is set.  With T == Tk <= 32 and the upper words zero this
 * is eagle_tree_attention_f16; the expansion has T = k queries and Tk = k * (level + 1) rows
 * (every earlier level's rows plus its own).  q [H,T,hd], out [T, H*hd]; the workspace is the
 * one of eagle_tree_attention_f16. */
int eagle_draft_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                              const uint32_t* mask_words, const int32_t* cache_len_dev, void* out,
                              int T, int Tk, int H, int G, int hd, long capacity, int max_len,
                              float scale, void* workspace, size_t workspace_bytes,
                              eagle_stream_t stream);

/* eagle_draft_attention_f16 for up to EAGLE_MAX_TREE_SLOTS query tokens, as the verification
 * forward (mlx_eagle.py:329-346 through mlx_llama.py:185-192) of a tree above 32 tokens needs
 * (the reference's default is 39 draft nodes, mlx_eagle.py:390,510; there Tk = T): T queries
 * against the P = *cache_len_dev prefix rows and the Tk <= 64 rows P .. P+Tk-1, of which query t
 * sees row j iff bit (j % 32) of mask_words[2*t + j/32] is set.  One launch pair: the queries go
 * in pieces of 32 rows over the same keys.  q [H,T,hd], out [T, H*hd]. */
size_t eagle_tree_attention_wide_workspace_bytes(int T, int H, int hd, int max_len);
int eagle_tree_attention_wide_f16(const void* q, const void* k_cache, const void* v_cache,
                                  const uint32_t* mask_words, const int32_t* cache_len_dev, void* out,
                                  int T, int Tk, int H, int G, int hd, long capacity, int max_len,
                                  float scale, void* workspace, size_t workspace_bytes,
                                  eagle_stream_t stream);

/* Causal attention of a prompt chunk (mlx_llama.py:185-192 with the causal mask of
 * mlx_llama.py:275-276; mlx_eagle.py:522-533): R query rows (a multiple of 32, at most
 * EAGLE_MAX_CHUNK) in pieces of 32.  Piece j has its rows at cache rows piece_len_dev[j] ..
 * piece_len_dev[j] + 31 (already appended), sees every cache row before them and its own rows
 * causally.  q [H,R,hd] (rotated), out [R, H*hd].  One launch pair for all pieces. */
size_t eagle_causal_attention_workspace_bytes(int R, int H, int hd, int max_len);
int eagle_causal_attention_f16(const void* q, const void* k_cache, const void* v_cache,
                               const int32_t* piece_len_dev, void* out, int R, int H, int G, int hd,
                               long capacity, int max_len, float scale, void* workspace,
                               size_t workspace_bytes, eagle_stream_t stream);

/* Row argmax of fp16 logits [R,V], lowest index among equal maxima
 * (mx.argmax at mlx_eagle.py:316,534,596).  out [R] int32. */
size_t eagle_argmax_workspace_bytes(int R, long V);
int eagle_argmax_rows_f16(const void* logits, int32_t* out, int R, long V,
                          void* workspace, size_t workspace_bytes, eagle_stream_t stream);

/* ---------------------------------------------------------------------------
 * Tree construction and acceptance (integer work, single workgroup kernels).
 * ------------------------------------------------------------------------- */

/* process_draft_tree (mlx_eagle.py:217-250): from C = k + k*k*depth candidate
 * scores (fp16, flat), their token ids and the parent table, pick the `total`
 * best (descending score, ties to the lowest flat index), order them by flat
 * index and emit
 *   tree_position_ids [T] int32, mask_index [total] int32, draft_tokens [T] int32,
 *   tree_mask_bits (ancestor-or-self rows): [T] uint32 for T = total + 1 <= 32, [T][2] uint32
 *   (low word, high word) for 32 < T <= EAGLE_MAX_TREE_SLOTS.
 * parents_list [C/k] uint32: 0 for the root's children, else parent flat id + 1.
 * sampled_token_dev: the root token. */
int eagle_process_draft_tree(const void* scores, const int32_t* tokens,
                             const uint32_t* parents_list, const int32_t* sampled_token_dev,
                             int C, int k, int total, int32_t* tree_position_ids,
                             int32_t* mask_index, int32_t* draft_tokens,
                             uint32_t* tree_mask_bits, eagle_stream_t stream);

/* post_process_draft_tree (mlx_eagle.py:254-295) without the host round trip:
 * retrieve_indices [64,64] int32 (row r = path of the r-th leaf, -1 padded; EAGLE_MAX_TREE_SLOTS
 * rows and columns whatever the tree size),
 * shape_out [2] int32 = {leaf_num, max_depth + 1}. */
int eagle_post_process_draft_tree(const int32_t* tree_position_ids, const int32_t* mask_index,
                                  int total, int32_t* retrieve_indices, int32_t* shape_out,
                                  eagle_stream_t stream);

/* Greedy acceptance (evaluate_posterior_greedy, mlx_eagle.py:311-326, with the
 * gathers of :582-589).  node_argmax [T] is the argmax token of each tree node's
 * logits, T <= EAGLE_MAX_TREE_SLOTS.  retrieve_indices [64,64] / shape as produced above; a -1
 * entry selects node T-1, as the reference's negative gather index does.
 * result [4 + 64] int32 = {best, accept_length, bonus_node, next_token,
 * accept_indices[0..accept_length)}; accepted_tokens [64] int32. */
int eagle_greedy_accept(const int32_t* node_argmax, const int32_t* draft_tokens,
                        const int32_t* retrieve_indices, const int32_t* shape, int T,
                        int32_t* result, int32_t* accepted_tokens, eagle_stream_t stream);

/* accept_candidate (mlx_eagle.py:349-376) for n_caches K or V buffers at once:
 * rows P + accept_indices[j] move to P + 1 + j for j < accept_length (gather
 * first, then scatter), then *cache_len_dev = min(P + accept_length + 1, capacity).
 * caches: device array of n_caches pointers to [G,capacity,hd] fp16 buffers.
 * accept [4 + 64] int32 in the layout of eagle_greedy_accept's result. */
int eagle_kv_compact_f16(void* const* caches_dev, int n_caches, const int32_t* accept,
                         int32_t* cache_len_dev, int G, int hd, long capacity,
                         eagle_stream_t stream);

/* ---------------------------------------------------------------------------
 * Draft-side tree expansion (generate_draft_tree and its helpers).
 * ------------------------------------------------------------------------- */

/* The k <= 8 most likely tokens of each of R <= 32 rows of fp16 logits [*, V] and their
 * log-probabilities in fp16, best first, equal scores lowest index first.  row_index (may be
 * NULL) selects the rows: row r reads logits row row_index[r] (a device value, e.g. the
 * accept length of mlx_eagle.py:404).
 *   mode 0 (mlx_eagle.py:410-412): top-k of the logits, score = fp16(logit - fp16(logsumexp))
 *   mode 1 (mlx_eagle.py:103-104): score = fp16(log(fp16(softmax))), top-k of the scores
 * (in fp16 distinct logits can share a score; the order among them is by index).
 * out_index [R,k] int32, out_score [R,k] fp16. */
size_t eagle_logsoftmax_topk_workspace_bytes(int R, long V);
int eagle_logsoftmax_topk_f16(const void* logits, const int32_t* row_index, int R, long V, int k,
                              int mode, int32_t* out_index, void* out_score, void* workspace,
                              size_t workspace_bytes, eagle_stream_t stream);

/* State of generate_draft_tree before its loop (mlx_eagle.py:130-155) from the level-0 top-k
 * (topk_index [k] int32, topk_score [k] fp16):
 *   saved_scores [k + k*k*depth] fp16 and saved_tokens (same length, int32): entries 0..k-1;
 *   parents [1 + k*depth] uint32: entry 0 = 0 and the level-0 rows 1..k = 1..k;
 *   cur_scores [k] fp16, cur_ids [k] int32: scores and input tokens of the first draft forward;
 *   mask_words [k][2] uint32: the identity block (query r sees expansion row r). */
int eagle_draft_tree_init(const int32_t* topk_index, const void* topk_score, int k,
                          void* saved_scores, int32_t* saved_tokens, uint32_t* parents,
                          void* cur_scores, int32_t* cur_ids, uint32_t* mask_words,
                          eagle_stream_t stream);

/* One level of the loop after the draft forward and the per-row top-k (mode 1) of its logits:
 * process_generate_tree_iteration (mlx_eagle.py:97-115) and the bookkeeping around it
 * (mlx_eagle.py:157-162,171,194-207).  topk_index / topk_score [k,k].  Writes the level's k*k
 * cumulative scores (fp16 add) and tokens into saved_scores / saved_tokens at k + k*k*level,
 * selects the k best (descending, ties lowest flat index) into topk_cs_index [k], out_ids [k]
 * (= topk_cs_index / k), cur_scores, cur_ids; unless it is the last level, parents rows
 * 1 + k*(level+1) .. and mask_words for the next level (child r inherits the words of query
 * out_ids[r] and sees expansion row k*(level+1) + r).  Needs k * depth <= 64. */
int eagle_draft_tree_level(const int32_t* topk_index, const void* topk_score, int level, int k,
                           int depth, void* saved_scores, int32_t* saved_tokens, uint32_t* parents,
                           void* cur_scores, int32_t* cur_ids, uint32_t* mask_words,
                           int32_t* out_ids, int32_t* topk_cs_index, eagle_stream_t stream);

/* Loop state of the speculative step on the device, so that consecutive steps need no host
 * round trip.  `accept` is the result array of eagle_greedy_accept of the previous step
 * ({best, accept_length, bonus_node, next_token, ...}).
 * eagle_spec_begin (mlx_eagle.py:393-394): *expand_len = *write_len = *draft_len + 1 +
 * accept_length, the row at which the expansion starts in the draft cache.
 * eagle_spec_update (mlx_eagle.py:591-599) after the verification: y [y_len] = the accepted
 * tokens, the bonus token, zeros; *draft_len = *expand_len; *root_token = the bonus token; the
 * accept_length + 1 new tokens are appended to out_tokens [max_out] at *out_count, which
 * advances (tokens beyond max_out are dropped, the count still advances). */
int eagle_spec_begin(const int32_t* draft_len_dev, const int32_t* accept, int32_t* expand_len_dev,
                     int32_t* write_len_dev, eagle_stream_t stream);
int eagle_spec_update(const int32_t* accept, const int32_t* accepted_tokens, int32_t* y, int y_len,
                      int32_t* draft_len_dev, const int32_t* expand_len_dev, int32_t* root_token_dev,
                      int32_t* out_tokens, int32_t* out_count_dev, int max_out, eagle_stream_t stream);

/* Small device-side helpers for graph-replayed steps. */
int eagle_fill_i32(int32_t* dst, int32_t value, long n, eagle_stream_t stream);
/* positions[t] = *cache_len_dev + tree_position_ids[t] (mlx_eagle.py:343). */
int eagle_tree_positions(const int32_t* tree_position_ids, const int32_t* cache_len_dev,
                         int32_t* positions, int T, eagle_stream_t stream);
/* *cache_len_dev += delta (KVCache.offset bookkeeping after an append). */
int eagle_advance_len(int32_t* cache_len_dev, int delta, eagle_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* EAGLE_MI355X_H */
