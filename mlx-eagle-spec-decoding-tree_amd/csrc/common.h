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
