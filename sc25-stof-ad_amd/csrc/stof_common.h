// Shared device-side types and small helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "stof_abi.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define STOF_WAVE 64

// One wavefront spans two halves of 32 lanes; exchange a value with the partner lane
// (lane ^ 32).  Used by the 32x32 MFMA layouts where a column lives in lanes l and l^32.
__device__ __forceinline__ float xchg32(float x) {
  return __shfl_xor(x, 32, 64);
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

static inline int stof_check_launch() {
  return hipGetLastError() == hipSuccess ? STOF_OK : STOF_ERR_LAUNCH;
}

static inline bool stof_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
