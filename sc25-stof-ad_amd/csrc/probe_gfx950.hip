// Measurement probes of the library: the shader clock a kernel actually runs at, and the issue
// rates of the attention loop's instruction mix.  Nothing on the product path calls these; bench.py
// does, so that the figures its roofline fractions rest on are measured in the run that reports them.
#include "stof_common.h"

namespace {

// One wavefront spins for `iters` rounds of dependent integer adds between two readings of the
// shader cycle counter (s_memtime) and of the constant 100 MHz counter (s_memrealtime).
// out[0] = shader cycles, out[1] = 10 ns ticks: clock = out[0] / out[1] * 100 MHz.  Launched on a
// second stream while another kernel loads the chip, it reads the clock under that load.
__global__ __launch_bounds__(64) void probe_clock_kernel(unsigned long long* out, int iters) {
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  unsigned x = threadIdx.x;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int j = 0; j < 16; ++j) asm volatile("v_add_u32 %0, %0, 1" : "+v"(x));
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) { out[0] = c1 - c0; out[1] = r1 - r0; out[2] = x; }
}

}  // namespace

extern "C" int stof_probe_clock(unsigned long long* out3, int iters, void* stream) {
  if (!out3) return STOF_ERR_NULL_POINTER;
  if (iters <= 0 || iters > (1 << 24)) return STOF_ERR_BAD_SHAPE;
  hipLaunchKernelGGL(probe_clock_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, out3, iters);
  return stof_check_launch();
}

extern "C" int stof_device_compute_units(void) {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return STOF_ERR_LAUNCH;
  return n;
}
