// Measurement probes of the library: the shader clock a kernel actually runs at, and the issue
// rates of the attention loop's instruction mix.  Nothing on the product path calls these; bench.py
// does, so that the figures its roofline fractions rest on are measured in the run that reports them.
#include "stof_common.h"

extern "C" int stof_device_compute_units(void);

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

// The instruction mix of one step of the attention loop (32 queries x 64 keys per wavefront, head
// size 64) with everything but the arithmetic taken away: no global or LDS access, no barrier, no
// mask, no walk - operands sit in registers.  Per step: 8 MFMA 32x32x16 (scores), then per score
// one multiply-add and one exp2, per pair one convert and one packed add, 16 max3 and the lazy
// test of the running max, then 8 MFMA (second product).  PARTS: 1 = the MFMAs only, 2 = the
// vector arithmetic only (on scores kept in registers), 3 = both as the kernel issues them.
// What it measures is the issue-rate ceiling of that mix on a SIMD shared by `waves per SIMD`
// wavefronts; out[0..2] of workgroup 0: shader cycles and 10 ns ticks of its first wavefront.
template <int PARTS>
__global__ __launch_bounds__(256, 4) void probe_issue_mix_kernel(unsigned long long* out, float* sink, int steps, float c) {
  const int lane = threadIdx.x & 63;
  half8_t kf[4], qf[4], vf[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      kf[i][e] = (half_t)(0.01f * (float)((lane + 3 * i + e) & 15) - 0.07f);
      qf[i][e] = (half_t)(0.02f * (float)((lane + 5 * i + 2 * e) & 15) - 0.11f);
      vf[i][e] = (half_t)(0.03f * (float)((lane + 7 * i + 3 * e) & 15) - 0.2f);
    }
  floatx16 o0, o1, s0, s1;
#pragma unroll
  for (int r = 0; r < 16; ++r) { o0[r] = 0.f; o1[r] = 0.f; s0[r] = 0.01f * (float)(lane + r); s1[r] = -0.02f * (float)(lane - r); }
  float m_run = 0.5f, l_run = 0.f;
  const unsigned long long c0 = __builtin_readcyclecounter();
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < steps; ++it) {
    if (PARTS & 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) { s0[r] = 0.f; s1[r] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[ks], qf[ks], s1, 0, 0, 0);
      }
    }
    half8_t p0[2], p1[2];
    if (PARTS & 2) {
      float mx = s0[0];
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(fmaxf(mx, s0[r]), s1[r]);
      const unsigned u = __builtin_bit_cast(unsigned, mx);
      const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
      mx = fmaxf(__builtin_bit_cast(float, (unsigned)sw[0]), __builtin_bit_cast(float, (unsigned)sw[1]));
      if (__any(mx * c > m_run + 1.0e30f)) m_run = mx;      // (the lazy test; never taken here)
      half2_t part[4];
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[r], c, -m_run)), e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[r + 1], c, -m_run));
        const float f0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[r], c, -m_run)), f1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[r + 1], c, -m_run));
        const half2_t e2 = {(half_t)e0, (half_t)e1}, f2 = {(half_t)f0, (half_t)f1};
        p0[r >> 3][r & 7] = e2[0]; p0[r >> 3][(r & 7) + 1] = e2[1];
        p1[r >> 3][r & 7] = f2[0]; p1[r >> 3][(r & 7) + 1] = f2[1];
        const int i = (r >> 1) & 3;
        part[i] = r < 8 ? e2 + f2 : part[i] + e2 + f2;
      }
      const half2_t tot = (part[0] + part[1]) + (part[2] + part[3]);
      l_run += (float)tot[0] + (float)tot[1];
      m_run += 1e-30f * l_run;   // (the subtrahend moves with the loop, so that no exponential is hoisted out of it)
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) { p0[h] = qf[h]; p1[h] = qf[2 + h]; }
    }
    if (PARTS & 1) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        o0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[h], p0[h], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 + h], p0[h], o1, 0, 0, 0);
        o0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[h], p1[h], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[2 + h], p1[h], o1, 0, 0, 0);
      }
    }
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
  float acc = l_run + m_run;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc += o0[r] + o1[r] + s0[r] + s1[r];
  if (acc == 123.456f) sink[threadIdx.x] = acc;            // (never true: keeps the arithmetic alive)
  if (blockIdx.x == 0 && threadIdx.x == 0) { out[0] = c1 - c0; out[1] = r1 - r0; out[2] = (unsigned long long)steps; }
}

}  // namespace

extern "C" int stof_probe_issue_mix(int parts, int waves_per_simd, int steps, unsigned long long* out3, float* sink256, void* stream) {
  if (!out3 || !sink256) return STOF_ERR_NULL_POINTER;
  if (parts < 1 || parts > 3 || waves_per_simd < 1 || waves_per_simd > 4 || steps <= 0 || steps > (1 << 20)) return STOF_ERR_BAD_SHAPE;
  const int cus = stof_device_compute_units();
  if (cus <= 0) return STOF_ERR_LAUNCH;
  // a workgroup is four wavefronts, one per SIMD: `waves_per_simd` workgroups per compute unit
  const dim3 grid((unsigned)(cus * waves_per_simd)), block(256);
  hipStream_t st = (hipStream_t)stream;
  const float c = 0.18033688f;
  if (parts == 1) hipLaunchKernelGGL(probe_issue_mix_kernel<1>, grid, block, 0, st, out3, sink256, steps, c);
  else if (parts == 2) hipLaunchKernelGGL(probe_issue_mix_kernel<2>, grid, block, 0, st, out3, sink256, steps, c);
  else hipLaunchKernelGGL(probe_issue_mix_kernel<3>, grid, block, 0, st, out3, sink256, steps, c);
  return stof_check_launch();
}

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
