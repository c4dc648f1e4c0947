// Shared declarations for the gfx950 kernels behind include/eagle_mi355x.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/eagle_mi355x.h"

#define EAGLE_EXPORT extern "C" __attribute__((visibility("default")))

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

static inline bool eagle_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline int eagle_launch_status() {
  return hipGetLastError() == hipSuccess ? EAGLE_OK : EAGLE_ERR_HIP;
}

// Wave-wide reductions over 64 lanes.
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Rows of a partial tile of the slab form: 32 for up to 32 rows of x, 64 for 33..64.
__host__ __device__ inline int eagle_slab_rows(int M) { return M > 32 ? 64 : 32; }

// Eight consecutive values of a matmul result that is held as fp32 partial sums of K slabs
// (eagle_qmm_slab_partial_w4g64): fp16 of the sum in slab order, then the fp16 bias.  `at` is
// the element offset inside a slab, `stride` the elements per slab.  All loads are issued
// before the first add.
__device__ inline half8_t eagle_slab_sum8(const float* __restrict__ partial, int nslab, size_t stride,
                                          size_t at, const half_t* __restrict__ bias8) {
  float4_t lo = float4_t{0.f, 0.f, 0.f, 0.f}, hi = lo;
  const float* p = partial + at;
  for (int z = 0; z < nslab; z += 8) {
    float4_t a[8], c[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int zz = z + k < nslab ? z + k : nslab - 1;
      a[k] = *reinterpret_cast<const float4_t*>(p + (size_t)zz * stride);
      c[k] = *reinterpret_cast<const float4_t*>(p + (size_t)zz * stride + 4);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (z + k < nslab) {
        lo += a[k];
        hi += c[k];
      }
  }
  half8_t v = half8_t{(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3],
                      (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
  if (bias8) {
    const half8_t b8 = *reinterpret_cast<const half8_t*>(bias8);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = v[e] + b8[e];
  }
  return v;
}
