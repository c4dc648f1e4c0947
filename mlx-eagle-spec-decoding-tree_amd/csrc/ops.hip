// Element-wise and row-wise operators of the tree-verify forward (gfx950):
// arrayed-position RoPE, fused RoPE + KV append, RMSNorm (+ residual), SiLU*mul,
// residual add, quantised embedding gather, row argmax.
#include "common.h"

#include <math.h>

namespace {

// ------------------------------------------------------------------------------------
// RoPE, one integer position per (batch, token), half-split pairing, fp32 math.
// Reference: mlx_arrayed_rope_kernel.py:60-123.
// ------------------------------------------------------------------------------------
__device__ inline void rotate8(const half8_t lo, const half8_t hi, const float* inv_freq,
                               int i0, float scale, float pos, half8_t* olo, half8_t* ohi) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float lf = scale * inv_freq[i0 + j];
    const float theta = lf * pos;
    float sn, cs;
    sincosf(theta, &sn, &cs);
    const float x1 = (float)lo[j];
    const float x2 = (float)hi[j];
    // one fused multiply-add on an explicitly rounded product: every rotation in the library
    // uses this form, so that they agree bit for bit
    (*olo)[j] = (half_t)__builtin_fmaf(x1, cs, -(x2 * sn));
    (*ohi)[j] = (half_t)__builtin_fmaf(x1, sn, x2 * cs);
  }
}

// x, out: [B,H,L,hd]; one thread rotates 8 pairs.
__global__ void rope_arrayed_kernel(const half_t* __restrict__ x, const int32_t* __restrict__ pos,
                                    const float* __restrict__ inv_freq, float scale,
                                    half_t* __restrict__ out, int B, int H, int L, int hd) {
  const int half = hd >> 1;
  const int per_row = half >> 3;
  const long total = (long)B * H * L * per_row;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % per_row);
  const long row = idx / per_row;          // (b*H + h)*L + t
  const int t = (int)(row % L);
  const int b = (int)(row / ((long)H * L));
  const float p = (float)pos[(long)b * L + t];
  const half_t* xr = x + row * hd;
  half_t* orow = out + row * hd;
  const half8_t lo = *reinterpret_cast<const half8_t*>(xr + c * 8);
  const half8_t hi = *reinterpret_cast<const half8_t*>(xr + half + c * 8);
  half8_t olo, ohi;
  rotate8(lo, hi, inv_freq, c * 8, scale, p, &olo, &ohi);
  *reinterpret_cast<half8_t*>(orow + c * 8) = olo;
  *reinterpret_cast<half8_t*>(orow + half + c * 8) = ohi;
}

// Generic head sizes (hd/2 not a multiple of 8): one thread per pair.
__global__ void rope_arrayed_scalar_kernel(const half_t* __restrict__ x,
                                           const int32_t* __restrict__ pos,
                                           const float* __restrict__ inv_freq, float scale,
                                           half_t* __restrict__ out, int B, int H, int L, int hd) {
  const int half = hd >> 1;
  const long total = (long)B * H * L * half;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int i = (int)(idx % half);
  const long row = idx / half;
  const int t = (int)(row % L);
  const int b = (int)(row / ((long)H * L));
  const float lf = scale * inv_freq[i];
  const float theta = lf * (float)pos[(long)b * L + t];
  float sn, cs;
  sincosf(theta, &sn, &cs);
  const float x1 = (float)x[row * hd + i];
  const float x2 = (float)x[row * hd + i + half];
  out[row * hd + i] = (half_t)__builtin_fmaf(x1, cs, -(x2 * sn));
  out[row * hd + i + half] = (half_t)__builtin_fmaf(x1, sn, x2 * cs);
}

// Token-major projections -> rotated q [H,T,hd] and K/V cache rows P + t.
// grid.x covers T * (H + 2G) * (hd/16) threads.
__global__ void rope_kv_append_kernel(const half_t* __restrict__ q_lin,
                                      const half_t* __restrict__ k_lin,
                                      const half_t* __restrict__ v_lin,
                                      const int32_t* __restrict__ pos,
                                      const float* __restrict__ inv_freq, float scale,
                                      half_t* __restrict__ q_out, half_t* __restrict__ k_cache,
                                      half_t* __restrict__ v_cache,
                                      const int32_t* __restrict__ len_dev, int T, int H, int G,
                                      int hd, long cap, long ld_q, long ld_kv,
                                      const float* __restrict__ rope_cs) {
  const int half = hd >> 1;
  const int per_row = half >> 3;
  const int heads = H + 2 * G;
  const long total = (long)T * heads * per_row;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % per_row);
  const int hh = (int)((idx / per_row) % heads);
  const int t = (int)(idx / ((long)per_row * heads));
  const long P = *len_dev;
  if (P + t >= cap) return;   // host checks capacity; never write past the buffer
  if (hh < H + G) {
    const bool is_q = hh < H;
    const int head = is_q ? hh : hh - H;
    const half_t* src = is_q ? q_lin + t * ld_q + (long)head * hd : k_lin + t * ld_kv + (long)head * hd;
    half_t* dst = is_q ? q_out + ((long)head * T + t) * hd : k_cache + ((long)head * cap + P + t) * hd;
    const half8_t lo = *reinterpret_cast<const half8_t*>(src + c * 8);
    const half8_t hi = *reinterpret_cast<const half8_t*>(src + half + c * 8);
    half8_t olo, ohi;
    if (rope_cs) {
      // (cos, sin) of this token's angles from the per-step table: the same values, no sincosf
      const float4_t* cs = reinterpret_cast<const float4_t*>(rope_cs + ((long)t * half + c * 8) * 2);
#pragma unroll
      for (int j2 = 0; j2 < 4; ++j2) {
        const float4_t v = cs[j2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int j = 2 * j2 + e;
          const float co = v[2 * e], sn = v[2 * e + 1];
          const float x1 = (float)lo[j], x2 = (float)hi[j];
          olo[j] = (half_t)__builtin_fmaf(x1, co, -(x2 * sn));
          ohi[j] = (half_t)__builtin_fmaf(x1, sn, x2 * co);
        }
      }
    } else {
      rotate8(lo, hi, inv_freq, c * 8, scale, (float)pos[t], &olo, &ohi);
    }
    *reinterpret_cast<half8_t*>(dst + c * 8) = olo;
    *reinterpret_cast<half8_t*>(dst + half + c * 8) = ohi;
  } else {
    const int head = hh - H - G;
    const half_t* src = v_lin + t * ld_kv + (long)head * hd;
    half_t* dst = v_cache + ((long)head * cap + P + t) * hd;
    *reinterpret_cast<half8_t*>(dst + c * 8) = *reinterpret_cast<const half8_t*>(src + c * 8);
    *reinterpret_cast<half8_t*>(dst + half + c * 8) =
        *reinterpret_cast<const half8_t*>(src + half + c * 8);
  }
}

// The same with the fused q|k|v projection held as fp32 partial sums of nslab K slabs,
// [slab][32][(H + 2G) hd] with a row = [q heads | k heads | v heads]: every value is
// fp16(sum of the slabs) + bias before the rotation.  One thread per four column pairs
// (half of the work of a thread above, twice the threads: all its slab loads are in flight
// together and the launch is a few dozen workgroups either way).
__global__ void rope_kv_append_slabs_kernel(const float* __restrict__ partial, int nslab,
                                            const half_t* __restrict__ bias,
                                            const float* __restrict__ rope_cs,
                                            half_t* __restrict__ q_out, half_t* __restrict__ k_cache,
                                            half_t* __restrict__ v_cache,
                                            const int32_t* __restrict__ len_dev, int T, int H, int G,
                                            int hd, long cap) {
  const int half = hd >> 1;
  const int per_row = half >> 2;
  const int heads = H + 2 * G;
  const long total = (long)T * heads * per_row;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % per_row) * 4;
  const int hh = (int)((idx / per_row) % heads);
  const int t = (int)(idx / ((long)per_row * heads));
  const size_t ld = (size_t)heads * hd;
  const size_t stride = (size_t)eagle_slab_rows(T) * ld;
  const float* p = partial + (size_t)t * ld + (size_t)hh * hd + c;
  // the cache length, cos / sin and the bias are requested with the slabs
  const long P = *len_dev;
  float4_t cs0 = float4_t{0.f, 0.f, 0.f, 0.f}, cs1 = cs0;
  if (hh < H + G) {
    const float4_t* cs = reinterpret_cast<const float4_t*>(rope_cs + ((long)t * half + c) * 2);
    cs0 = cs[0];
    cs1 = cs[1];
  }
  half4_t blo = half4_t{0, 0, 0, 0}, bhi = blo;
  if (bias) {
    blo = *reinterpret_cast<const half4_t*>(bias + (size_t)hh * hd + c);
    bhi = *reinterpret_cast<const half4_t*>(bias + (size_t)hh * hd + half + c);
  }
  float4_t lo = float4_t{0.f, 0.f, 0.f, 0.f}, hi = lo;
  for (int z = 0; z < nslab; z += 8) {
    float4_t a[8], b[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int zz = z + k < nslab ? z + k : nslab - 1;
      a[k] = *reinterpret_cast<const float4_t*>(p + (size_t)zz * stride);
      b[k] = *reinterpret_cast<const float4_t*>(p + (size_t)zz * stride + half);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (z + k < nslab) {
        lo += a[k];
        hi += b[k];
      }
  }
  half4_t xlo, xhi;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    xlo[j] = (half_t)lo[j];
    xhi[j] = (half_t)hi[j];
  }
  if (bias) {
    xlo += blo;
    xhi += bhi;
  }
  if (P + t >= cap) return;   // host checks capacity; never write past the buffer
  if (hh < H + G) {
    const bool is_q = hh < H;
    const int head = is_q ? hh : hh - H;
    half_t* dst = is_q ? q_out + ((long)head * T + t) * hd : k_cache + ((long)head * cap + P + t) * hd;
    half4_t olo, ohi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float co = j < 2 ? cs0[2 * j] : cs1[2 * (j - 2)];
      const float sn = j < 2 ? cs0[2 * j + 1] : cs1[2 * (j - 2) + 1];
      const float x1 = (float)xlo[j], x2 = (float)xhi[j];
      olo[j] = (half_t)__builtin_fmaf(x1, co, -(x2 * sn));
      ohi[j] = (half_t)__builtin_fmaf(x1, sn, x2 * co);
    }
    *reinterpret_cast<half4_t*>(dst + c) = olo;
    *reinterpret_cast<half4_t*>(dst + half + c) = ohi;
  } else {
    half_t* dst = v_cache + ((long)(hh - H - G) * cap + P + t) * hd;
    *reinterpret_cast<half4_t*>(dst + c) = xlo;
    *reinterpret_cast<half4_t*>(dst + half + c) = xhi;
  }
}

// ------------------------------------------------------------------------------------
// RMSNorm with optional residual add; one 256-thread workgroup per row, the row stays
// in registers between the two passes.  D % 8 == 0, D <= 256 * 8 * RMS_MAXV.
// ------------------------------------------------------------------------------------
constexpr int RMS_MAXV = 4;

// BLOCK threads per row; the norm weights are requested together with the row, before the
// reduction, so that their latency is not added to it.
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void rmsnorm_kernel(const half_t* __restrict__ x,
                                                        const half_t* __restrict__ res,
                                                        const half_t* __restrict__ w, float eps,
                                                        half_t* __restrict__ h_out,
                                                        half_t* __restrict__ out, int D,
                                                        const float* __restrict__ partial, int nslab) {
  // partial != nullptr: x is held as fp32 partial sums of nslab K slabs, [slab][32 or 64][D]
  // (64 when the launch has more than 32 rows)
  constexpr int NV = 256 * RMS_MAXV / BLOCK;     // vectors per thread
  __shared__ float red[BLOCK / 64];
  const int t = blockIdx.x;
  const int nvec = D >> 3;
  const half_t* xr = x + (long)t * D;
  half8_t v[NV], w8[NV];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * BLOCK;
    if (c < nvec) {
      w8[i] = *reinterpret_cast<const half8_t*>(w + c * 8);
      half8_t r8;
      if (res) r8 = *reinterpret_cast<const half8_t*>(res + (long)t * D + c * 8);
      half8_t a;
      if (partial)
        a = eagle_slab_sum8(partial, nslab, (size_t)eagle_slab_rows(gridDim.x) * D, (size_t)t * D + c * 8, nullptr);
      else
        a = *reinterpret_cast<const half8_t*>(xr + c * 8);
      if (res) {
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = (half_t)((float)a[j] + (float)r8[j]);
        *reinterpret_cast<half8_t*>(h_out + (long)t * D + c * 8) = a;
      }
      v[i] = a;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)a[j] * (float)a[j];
    }
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int k = 0; k < BLOCK / 64; ++k) tot += red[k];
  const float rinv = 1.0f / sqrtf(tot / (float)D + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * BLOCK;
    if (c < nvec) {
      half8_t o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (half_t)((float)w8[i][j] * ((float)v[i][j] * rinv));
      *reinterpret_cast<half8_t*>(out + (long)t * D + c * 8) = o;
    }
  }
}

// out = fp16(fp16(silu(g)) * u); g/u rows have stride `ld` (2*I when fused, I otherwise).
__global__ void silu_mul_kernel(const half_t* __restrict__ g, const half_t* __restrict__ u,
                                half_t* __restrict__ out, int T, int I, long ld) {
  const int per_row = I >> 3;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)T * per_row) return;
  const int c = (int)(idx % per_row);
  const long t = idx / per_row;
  const half8_t gv = *reinterpret_cast<const half8_t*>(g + t * ld + c * 8);
  const half8_t uv = *reinterpret_cast<const half8_t*>(u + t * ld + c * 8);
  half8_t o;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float x = (float)gv[j];
    const half_t a = (half_t)(x / (1.0f + expf(-x)));
    o[j] = (half_t)((float)a * (float)uv[j]);
  }
  *reinterpret_cast<half8_t*>(out + t * I + c * 8) = o;
}

__global__ void add_kernel(const half_t* __restrict__ a, const half_t* __restrict__ b,
                           half_t* __restrict__ out, long n) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i + 8 <= n) {
    const half8_t x = *reinterpret_cast<const half8_t*>(a + i);
    const half8_t y = *reinterpret_cast<const half8_t*>(b + i);
    half8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (half_t)((float)x[j] + (float)y[j]);
    *reinterpret_cast<half8_t*>(out + i) = o;
  } else {
    for (long j = i; j < n; ++j) out[j] = (half_t)((float)a[j] + (float)b[j]);
  }
}

// Embedding rows: one thread expands one packed word.
__global__ void embed_kernel(const int32_t* __restrict__ ids, const uint32_t* __restrict__ w,
                             const half_t* __restrict__ s, const half_t* __restrict__ b,
                             half_t* __restrict__ out, int T, int D, int V) {
  const int words = D >> 3;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)T * words) return;
  const int j = (int)(idx % words);
  const int t = (int)(idx / words);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);   // host validates ids it can see; stay in bounds
  const uint32_t word = w[(long)id * words + j];
  const float sc = (float)s[(long)id * (D >> 6) + (j >> 3)];
  const float bi = (float)b[(long)id * (D >> 6) + (j >> 3)];
  half8_t o;
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (half_t)__builtin_fmaf(sc, (float)((word >> (4 * i)) & 15u), bi);
  *reinterpret_cast<half8_t*>(out + (long)t * D + j * 8) = o;
}

// ------------------------------------------------------------------------------------
// Row argmax, first maximum.  Stage 1: grid (chunks, rows); stage 2: one wave per row.
// ------------------------------------------------------------------------------------
struct ValIdx {
  float v;
  int i;
};
__device__ inline ValIdx better(ValIdx a, ValIdx b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}
__device__ inline ValIdx wave_best(ValIdx a) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ValIdx b;
    b.v = __shfl_xor(a.v, o, 64);
    b.i = __shfl_xor(a.i, o, 64);
    a = better(a, b);
  }
  return a;
}

constexpr int ARGMAX_CHUNKS = 16;

__global__ __launch_bounds__(256) void argmax_stage1(const half_t* __restrict__ logits,
                                                     float* __restrict__ pv, int* __restrict__ pi,
                                                     long V) {
  __shared__ ValIdx red[4];
  const int row = blockIdx.y;
  const int ch = blockIdx.x;
  const long per = ((V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS + 7) / 8 * 8;
  const long beg = (long)ch * per;
  const long end = beg + per < V ? beg + per : V;
  const half_t* r = logits + (long)row * V;
  ValIdx best{-INFINITY, 0x7fffffff};
  const bool vec_ok = ((V & 7) == 0);
  if (vec_ok) {
    for (long i = beg + (long)threadIdx.x * 8; i < end; i += 256 * 8) {
      const half8_t v = *reinterpret_cast<const half8_t*>(r + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) best = better(best, ValIdx{(float)v[j], (int)(i + j)});
    }
  } else {
    for (long i = beg + threadIdx.x; i < end; i += 256)
      best = better(best, ValIdx{(float)r[i], (int)i});
  }
  best = wave_best(best);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    ValIdx b = better(better(red[0], red[1]), better(red[2], red[3]));
    pv[row * ARGMAX_CHUNKS + ch] = b.v;
    pi[row * ARGMAX_CHUNKS + ch] = b.i;
  }
}

__global__ void argmax_stage2(const float* __restrict__ pv, const int* __restrict__ pi,
                              int32_t* __restrict__ out) {
  const int row = blockIdx.x;
  ValIdx b{-INFINITY, 0x7fffffff};
  if (threadIdx.x < ARGMAX_CHUNKS)
    b = ValIdx{pv[row * ARGMAX_CHUNKS + threadIdx.x], pi[row * ARGMAX_CHUNKS + threadIdx.x]};
  b = wave_best(b);
  if (threadIdx.x == 0) out[row] = b.i == 0x7fffffff ? 0 : b.i;
}

inline unsigned blocks_for(long n, int threads) { return (unsigned)((n + threads - 1) / threads); }

}  // namespace

EAGLE_EXPORT int eagle_rope_arrayed_f16(const void* x, const int32_t* positions,
                                        const float* inv_freqs, float scaling_factor, void* out,
                                        int B, int H, int L, int hd, eagle_stream_t stream) {
  if (!x || !positions || !inv_freqs || !out) return EAGLE_ERR_NULL;
  if (B < 1 || H < 1 || L < 1 || hd < 2 || (hd & 1)) return EAGLE_ERR_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int half = hd / 2;
  if ((half % 8) == 0 && eagle_aligned16(x) && eagle_aligned16(out)) {
    const long total = (long)B * H * L * (half / 8);
    hipLaunchKernelGGL(rope_arrayed_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, st,
                       (const half_t*)x, positions, inv_freqs, scaling_factor, (half_t*)out, B, H,
                       L, hd);
  } else {
    const long total = (long)B * H * L * half;
    hipLaunchKernelGGL(rope_arrayed_scalar_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, st,
                       (const half_t*)x, positions, inv_freqs, scaling_factor, (half_t*)out, B, H,
                       L, hd);
  }
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_rope_kv_append_f16(const void* q_lin, const void* k_lin, const void* v_lin,
                                          const int32_t* positions, const float* inv_freqs,
                                          float scaling_factor, void* q_out, void* k_cache,
                                          void* v_cache, const int32_t* cache_len_dev, int T,
                                          int H, int G, int hd, long capacity, long row_stride,
                                          eagle_stream_t stream) {
  if (!q_lin || !k_lin || !v_lin || !positions || !inv_freqs || !q_out || !k_cache || !v_cache ||
      !cache_len_dev)
    return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_TREE || H < 1 || G < 1 || (H % G) != 0 || hd < 16 || (hd % 16) != 0 ||
      capacity < T || row_stride < 0 || (row_stride % 8) != 0 ||
      (row_stride > 0 && row_stride < (long)H * hd))
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q_lin) || !eagle_aligned16(k_lin) || !eagle_aligned16(v_lin) ||
      !eagle_aligned16(q_out) || !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache))
    return EAGLE_ERR_ALIGN;
  const long total = (long)T * (H + 2 * G) * (hd / 16);
  hipLaunchKernelGGL(rope_kv_append_kernel, dim3(blocks_for(total, 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), (const half_t*)q_lin, (const half_t*)k_lin,
                     (const half_t*)v_lin, positions, inv_freqs, scaling_factor, (half_t*)q_out,
                     (half_t*)k_cache, (half_t*)v_cache, cache_len_dev, T, H, G, hd, capacity,
                     row_stride ? row_stride : (long)H * hd, row_stride ? row_stride : (long)G * hd,
                     (const float*)nullptr);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_rope_kv_append_table_f16(const void* q_lin, const void* k_lin,
                                                const void* v_lin, const float* rope_cs,
                                                void* q_out, void* k_cache, void* v_cache,
                                                const int32_t* cache_len_dev, int T, int H, int G,
                                                int hd, long capacity, long row_stride,
                                                eagle_stream_t stream) {
  if (!q_lin || !k_lin || !v_lin || !rope_cs || !q_out || !k_cache || !v_cache || !cache_len_dev)
    return EAGLE_ERR_NULL;
  if (T < 1 || T > EAGLE_MAX_CHUNK || H < 1 || G < 1 || (H % G) != 0 || hd < 16 || (hd % 16) != 0 ||
      capacity < T || row_stride < 0 || (row_stride % 8) != 0 ||
      (row_stride > 0 && row_stride < (long)H * hd))
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(q_lin) || !eagle_aligned16(k_lin) || !eagle_aligned16(v_lin) ||
      !eagle_aligned16(rope_cs) || !eagle_aligned16(q_out) || !eagle_aligned16(k_cache) ||
      !eagle_aligned16(v_cache))
    return EAGLE_ERR_ALIGN;
  const long total = (long)T * (H + 2 * G) * (hd / 16);
  hipLaunchKernelGGL(rope_kv_append_kernel, dim3(blocks_for(total, 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), (const half_t*)q_lin, (const half_t*)k_lin,
                     (const half_t*)v_lin, (const int32_t*)nullptr, (const float*)nullptr, 1.0f,
                     (half_t*)q_out, (half_t*)k_cache, (half_t*)v_cache, cache_len_dev, T, H, G, hd,
                     capacity, row_stride ? row_stride : (long)H * hd,
                     row_stride ? row_stride : (long)G * hd, rope_cs);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_rope_kv_append_slabs_f16(const float* partial, int slabs, const void* bias,
                                                const float* rope_cs, void* q_out, void* k_cache,
                                                void* v_cache, const int32_t* cache_len_dev, int T,
                                                int H, int G, int hd, long capacity,
                                                eagle_stream_t stream) {
  if (!partial || !rope_cs || !q_out || !k_cache || !v_cache || !cache_len_dev) return EAGLE_ERR_NULL;
  if (slabs < 1 || T < 1 || T > 64 || H < 1 || G < 1 || (H % G) != 0 || hd < 16 || (hd % 16) != 0 ||
      capacity < T)
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(partial) || !eagle_aligned16(rope_cs) || !eagle_aligned16(q_out) ||
      !eagle_aligned16(k_cache) || !eagle_aligned16(v_cache) || (bias && !eagle_aligned16(bias)))
    return EAGLE_ERR_ALIGN;
  const long total = (long)T * (H + 2 * G) * (hd / 8);
  hipLaunchKernelGGL(rope_kv_append_slabs_kernel, dim3(blocks_for(total, 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), partial, slabs, (const half_t*)bias, rope_cs,
                     (half_t*)q_out, (half_t*)k_cache, (half_t*)v_cache, cache_len_dev, T, H, G, hd,
                     capacity);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_rmsnorm_f16(const void* x, const void* residual, const void* w, float eps,
                                   void* h_out, void* out, int T, int D, eagle_stream_t stream) {
  if (!x || !w || !out || (residual && !h_out)) return EAGLE_ERR_NULL;
  if (T < 1 || D < 8 || (D % 8) != 0 || D > 256 * 8 * RMS_MAXV) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(w) || !eagle_aligned16(out) ||
      (residual && (!eagle_aligned16(residual) || !eagle_aligned16(h_out))))
    return EAGLE_ERR_ALIGN;
  if (D > 256 * 8)   // one vector per thread while the row is short enough
    hipLaunchKernelGGL(rmsnorm_kernel<512>, dim3(T), dim3(512), 0, static_cast<hipStream_t>(stream),
                       (const half_t*)x, (const half_t*)residual, (const half_t*)w, eps,
                       (half_t*)h_out, (half_t*)out, D, (const float*)nullptr, 0);
  else
    hipLaunchKernelGGL(rmsnorm_kernel<256>, dim3(T), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const half_t*)x, (const half_t*)residual, (const half_t*)w, eps,
                       (half_t*)h_out, (half_t*)out, D, (const float*)nullptr, 0);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_rmsnorm_slabs_f16(const float* partial, int slabs, const void* residual,
                                         const void* w, float eps, void* h_out, void* out, int T, int D,
                                         eagle_stream_t stream) {
  if (!partial || !w || !out || (residual && !h_out)) return EAGLE_ERR_NULL;
  if (slabs < 1 || T < 1 || T > 64 || D < 8 || (D % 8) != 0 || D > 256 * 8 * RMS_MAXV) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(partial) || !eagle_aligned16(w) || !eagle_aligned16(out) ||
      (residual && (!eagle_aligned16(residual) || !eagle_aligned16(h_out))))
    return EAGLE_ERR_ALIGN;
  if (D > 256 * 8)
    hipLaunchKernelGGL(rmsnorm_kernel<512>, dim3(T), dim3(512), 0, static_cast<hipStream_t>(stream),
                       (const half_t*)nullptr, (const half_t*)residual, (const half_t*)w, eps,
                       (half_t*)h_out, (half_t*)out, D, partial, slabs);
  else
    hipLaunchKernelGGL(rmsnorm_kernel<256>, dim3(T), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const half_t*)nullptr, (const half_t*)residual, (const half_t*)w, eps,
                       (half_t*)h_out, (half_t*)out, D, partial, slabs);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_silu_mul_f16(const void* gate, const void* up, void* out, int T, int I,
                                    eagle_stream_t stream) {
  if (!gate || !out) return EAGLE_ERR_NULL;
  if (T < 1 || I < 8 || (I % 8) != 0) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(gate) || !eagle_aligned16(out) || (up && !eagle_aligned16(up)))
    return EAGLE_ERR_ALIGN;
  const half_t* g = (const half_t*)gate;
  const half_t* u = up ? (const half_t*)up : g + I;
  const long ld = up ? I : 2L * I;
  const long total = (long)T * (I / 8);
  hipLaunchKernelGGL(silu_mul_kernel, dim3(blocks_for(total, 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), g, u, (half_t*)out, T, I, ld);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_add_f16(const void* a, const void* b, void* out, long n,
                               eagle_stream_t stream) {
  if (!a || !b || !out) return EAGLE_ERR_NULL;
  if (n < 1) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(a) || !eagle_aligned16(b) || !eagle_aligned16(out)) return EAGLE_ERR_ALIGN;
  hipLaunchKernelGGL(add_kernel, dim3(blocks_for((n + 7) / 8, 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), (const half_t*)a, (const half_t*)b,
                     (half_t*)out, n);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_embed_w4g64_f16(const int32_t* ids, const uint32_t* wq, const void* scales,
                                       const void* biases, void* out, int T, int D, int V,
                                       eagle_stream_t stream) {
  if (!ids || !wq || !scales || !biases || !out) return EAGLE_ERR_NULL;
  if (T < 1 || V < 1 || D < 64 || (D % 64) != 0) return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(out)) return EAGLE_ERR_ALIGN;
  const long total = (long)T * (D / 8);
  hipLaunchKernelGGL(embed_kernel, dim3(blocks_for(total, 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), ids, wq, (const half_t*)scales,
                     (const half_t*)biases, (half_t*)out, T, D, V);
  return eagle_launch_status();
}

EAGLE_EXPORT size_t eagle_argmax_workspace_bytes(int R, long V) {
  (void)V;
  if (R < 1) return 0;
  return (size_t)R * ARGMAX_CHUNKS * (sizeof(float) + sizeof(int));
}

EAGLE_EXPORT int eagle_argmax_rows_f16(const void* logits, int32_t* out, int R, long V,
                                       void* workspace, size_t workspace_bytes,
                                       eagle_stream_t stream) {
  if (!logits || !out) return EAGLE_ERR_NULL;
  if (R < 1 || R > 65535 || V < 1 || V > 0x7ffffff0L) return EAGLE_ERR_SHAPE;
  if (!workspace || workspace_bytes < eagle_argmax_workspace_bytes(R, V)) return EAGLE_ERR_WORKSPACE;
  if ((V % 8) == 0 && !eagle_aligned16(logits)) return EAGLE_ERR_ALIGN;
  float* pv = static_cast<float*>(workspace);
  int* pi = reinterpret_cast<int*>(pv + (size_t)R * ARGMAX_CHUNKS);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(argmax_stage1, dim3(ARGMAX_CHUNKS, R), dim3(256), 0, st,
                     (const half_t*)logits, pv, pi, V);
  hipLaunchKernelGGL(argmax_stage2, dim3(R), dim3(64), 0, st, pv, pi, out);
  return eagle_launch_status();
}
