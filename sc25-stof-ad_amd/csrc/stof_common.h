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

// BF: the tensors are bfloat16 instead of fp16.  Operand fragments are carried as 16-bit
// patterns in half_t / half8_t either way (loads, LDS and the transposing read do not look at
// the format); only the MFMA opcode and the conversions from and to fp32 differ.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
template <bool BF>
__device__ __forceinline__ floatx16 mfma32(half8_t a, half8_t b, floatx16 c) {
  if constexpr (BF)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// fp32 -> the tensors' 16-bit format (round to nearest even), as a 16-bit pattern in half_t
template <bool BF>
__device__ __forceinline__ half_t to_elem(float x) {
  if constexpr (BF) return __builtin_bit_cast(half_t, (__bf16)x);
  else return (half_t)x;
}
// the tensors' 16-bit format -> fp32 (bfloat16: the pattern is the upper half of the fp32 pattern)
template <bool BF>
__device__ __forceinline__ float from_elem(half_t e) {
  if constexpr (BF) return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(unsigned short, e) << 16);
  else return (float)e;
}

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

// GELU(x) = x * Phi(x), Phi the standard normal distribution function.  Both variants are
// evaluated as x * sigmoid(p(x)) = x / (1 + exp2(-log2(e) p(x))) with p an odd polynomial:
//  * erf form (torch approximate="none"): p(x) = x (a0 + a1 x^2 + a2 x^4), the coefficients a
//    weighted least-squares fit of x * sigmoid(p(x)) to x * Phi(x) that levels the error over
//    |x| <= 9: |error| <= 2.6e-5 everywhere (a fifth of the spacing of the fp16 output at the
//    argument where it peaks, x = -0.56), against 4.7e-4 for the tanh formula.  x^2 is held at
//    81 (a2 < 0, so p would turn round at |x| = 11; beyond 9 the sigmoid is 0 or 1 in fp32).
//    One reciprocal, one exp2, seven multiply-adds: half the instructions of an erf evaluation
//    (Abramowitz-Stegun 7.1.26: 17), which is what the epilogue of the FFN GEMM spends its time on;
//  * tanh form (approximate="tanh"): 0.5 x (1 + tanh(u)) = x * sigmoid(2u) exactly,
//    u = sqrt(2/pi) (x + 0.044715 x^3), i.e. p(x) = x (2 sqrt(2/pi) + 2 sqrt(2/pi) 0.044715 x^2).
__device__ __forceinline__ float stof_gelu_erf(float x) {
  constexpr float kNegLog2e = -1.4426950408889634f;
  constexpr float a0 = 1.5950157578067197f, a1 = 0.07401130113566103f, a2 = -0.0007030349551266337f;
  const float x2 = fminf(x * x, 81.0f);
  const float q = x * __builtin_fmaf(x2, __builtin_fmaf(x2, kNegLog2e * a2, kNegLog2e * a1), kNegLog2e * a0);
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(q));
}
__device__ __forceinline__ float stof_gelu_tanh(float x) {
  constexpr float k0 = -1.4426950408889634f * 2.0f * 0.7978845608028654f;
  const float q = x * __builtin_fmaf(x * x, k0 * 0.044715f, k0);
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(q));
}
// Activation selector of the GEMM epilogues (STOF_ACT_*).
template <int ACT> __device__ __forceinline__ float activate(float x) {
  if (ACT == STOF_ACT_GELU_ERF) return stof_gelu_erf(x);
  if (ACT == STOF_ACT_GELU_TANH) return stof_gelu_tanh(x);
  if (ACT == STOF_ACT_RELU) return fmaxf(x, 0.f);
  return x;
}

// Output rows written THROUGH the XCD's L2 at device scope (sc1): for tiles nobody in the launch
// reads again.  As plain cached stores they sit in L2 until the end-of-kernel write-back, which
// the next launch waits for.  The store is a raw buffer store (cache policy as an argument of
// the builtin), addressed as a wave-uniform base plus a 32-bit byte offset per lane.  (Written
// as inline assembly it loses the compiler's hazard handling: a 16-byte store whose data
// registers are overwritten within two instructions stores the new values for some lanes.)
typedef unsigned int uintx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stof_wave_rsrc(const void* wave_uniform_base) {
  const uint64_t a = reinterpret_cast<uint64_t>(wave_uniform_base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0, 0x7fffffff, 0x00020000);
}
constexpr int kStoreThrough = 16;   // cache-policy bits of the buffer builtins on gfx940+: 1 = sc0, 2 = nt, 16 = sc1
__device__ __forceinline__ void stof_store16_through(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset, half8_t v) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4_t, v), rsrc, (int)byte_offset, 0, kStoreThrough);
}

static inline int stof_check_launch() {
  return hipGetLastError() == hipSuccess ? STOF_OK : STOF_ERR_LAUNCH;
}

static inline bool stof_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
