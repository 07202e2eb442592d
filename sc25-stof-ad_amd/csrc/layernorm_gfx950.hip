// bias + residual + LayerNorm for gfx950: y = LN(x + bias + residual) * gamma + beta.
//
// Replaces batched_bias_layer_norm_fused_kernel (src/triton_template/add_layernorm.py:19-84),
// which walks each row three times from global memory.  Here one wavefront owns one row,
// reads it once with 16-byte loads, keeps it in registers for the exact two-pass
// mean / variance, and writes it once: the kernel moves the algorithmic minimum of bytes
// and is bound by HBM bandwidth.
#include "stof_common.h"

namespace {

struct LnParams {
  const half_t* x; const half_t* bias; const half_t* res; const half_t* gamma; const half_t* beta;
  half_t* y; float* mean; float* rstd;
  int64_t M; int N; float eps; float inv_n;
};

template <bool BF>
__device__ __forceinline__ void load8(const half_t* p, float (&v)[8]) {
  const half8_t h = *reinterpret_cast<const half8_t*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) { const half_t e = h[i]; v[i] = from_elem<BF>(e); }
}

// CH = 16-byte chunks per lane; the row has at most 64*CH chunks (N <= 512*CH).
// Every load of the row (x, residual, bias for all of the lane's chunks) is issued before the
// first value is converted, so a wave has 2-3 x CH 16-byte loads in flight instead of one: with
// one wave per row of 1.5 KB that is what it takes to keep HBM busy.  A chunk past the end of
// the row reads chunk 0 instead (a valid address) and is zeroed afterwards.
// BF: the tensors are bfloat16 instead of fp16 (statistics are fp32 either way).
template <int CH, bool BF = false>
__global__ __launch_bounds__(256) void bias_res_ln_kernel(const LnParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.M) return;
  const int nchunk = p.N >> 3;
  const half_t* xr = p.x + row * p.N;
  const half_t* rr = p.res ? p.res + row * p.N : nullptr;

  half8_t hx[CH], hr[CH], hb[CH];
  bool valid[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ch = lane + 64 * c;
    valid[c] = ch < nchunk;
    const int chs = valid[c] ? ch : 0;
    hx[c] = *reinterpret_cast<const half8_t*>(xr + 8 * chs);
    if (rr) hr[c] = *reinterpret_cast<const half8_t*>(rr + 8 * chs);
    if (p.bias) hb[c] = *reinterpret_cast<const half8_t*>(p.bias + 8 * chs);
  }
  float v[CH][8];
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const half_t xe = hx[c][i];
      float t = from_elem<BF>(xe);
      if (p.bias) { const half_t be = hb[c][i]; t += from_elem<BF>(be); }
      if (rr) { const half_t re = hr[c][i]; t += from_elem<BF>(re); }
      v[c][i] = valid[c] ? t : 0.f;
      s += v[c][i];
    }
  }
  const float mean = wave_sum(s) * p.inv_n;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c)
    if (valid[c]) {
#pragma unroll
      for (int i = 0; i < 8; ++i) { const float d = v[c][i] - mean; q += d * d; }
    }
  const float var = wave_sum(q) * p.inv_n;
  const float rstd = 1.0f / sqrtf(var + p.eps);
  if (lane == 0) {
    if (p.mean) p.mean[row] = mean;
    if (p.rstd) p.rstd[row] = rstd;
  }
  half_t* yr = p.y + row * p.N;
  const __amdgpu_buffer_rsrc_t y_rsrc = stof_wave_rsrc(yr);   // this wave's row
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int ch = lane + 64 * c;
    if (valid[c]) {
      float gm[8], bt[8];
      if (p.gamma) load8<BF>(p.gamma + 8 * ch, gm);
      if (p.beta) load8<BF>(p.beta + 8 * ch, bt);
      half8_t o;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = (v[c][i] - mean) * rstd;
        if (p.gamma) t *= gm[i];
        if (p.beta) t += bt[i];
        o[i] = to_elem<BF>(t);
      }
      stof_store16_through(y_rsrc, 16 * ch, o);
    }
  }
}

}  // namespace

extern "C" int stof_bias_res_ln_dt(const void* x, const void* bias, const void* residual,
                                   const void* gamma, const void* beta, void* y,
                                   float* mean, float* rstd,
                                   int64_t M, int64_t N, float eps, int dtype, void* stream) {
  if (!x || !y) return STOF_ERR_NULL_POINTER;
  if (dtype != STOF_DTYPE_F16 && dtype != STOF_DTYPE_BF16) return STOF_ERR_UNSUPPORTED;
  if (M <= 0 || N <= 0 || N % 8 != 0 || N > 8192 || M > ((int64_t)1 << 31)) return STOF_ERR_BAD_SHAPE;
  if (!stof_aligned16(x) || !stof_aligned16(y) || !stof_aligned16(bias) || !stof_aligned16(residual) ||
      !stof_aligned16(gamma) || !stof_aligned16(beta))
    return STOF_ERR_MISALIGNED;
  LnParams p;
  p.x = (const half_t*)x; p.bias = (const half_t*)bias; p.res = (const half_t*)residual;
  p.gamma = (const half_t*)gamma; p.beta = (const half_t*)beta; p.y = (half_t*)y;
  p.mean = mean; p.rstd = rstd; p.M = M; p.N = (int)N; p.eps = eps; p.inv_n = 1.0f / (float)N;
  const dim3 grid((unsigned)((M + 3) / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define STOF_LN_LAUNCH(CH) \
  do { \
    if (dtype == STOF_DTYPE_BF16) hipLaunchKernelGGL((bias_res_ln_kernel<CH, true>), grid, block, 0, st, p); \
    else hipLaunchKernelGGL((bias_res_ln_kernel<CH, false>), grid, block, 0, st, p); \
  } while (0)
  if (N <= 512) STOF_LN_LAUNCH(1);
  else if (N <= 1024) STOF_LN_LAUNCH(2);
  else if (N <= 2048) STOF_LN_LAUNCH(4);
  else if (N <= 4096) STOF_LN_LAUNCH(8);
  else STOF_LN_LAUNCH(16);
#undef STOF_LN_LAUNCH
  return stof_check_launch();
}

extern "C" int stof_bias_res_ln(const void* x, const void* bias, const void* residual,
                                const void* gamma, const void* beta, void* y,
                                float* mean, float* rstd,
                                int64_t M, int64_t N, float eps, void* stream) {
  return stof_bias_res_ln_dt(x, bias, residual, gamma, beta, y, mean, rstd, M, N, eps, STOF_DTYPE_F16, stream);
}
