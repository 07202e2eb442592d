// Chained GEMM + bias + activation + GEMM in one launch, for gfx950 (MI355X):
//   Y[M,H] = act(X[M,K] @ W1^T + b1[F]) @ W2^T (+ b2[H])        W1 as W1t[F,K], W2 as W2t[H,F]
// the reference's triton_matmul_batch (src/triton_template/gemm_gemm.py:99-174): the [M,F]
// intermediate (F = 4 x hidden in the encoder) never reaches HBM.
//
// The reference gives one program a block of output rows x output columns and recomputes the
// first product for every output column block.  Here the F dimension is what is split:
// workgroup (row block of 64 tokens, chunk of 128 intermediate features)
//   1. forms its 64 x 128 piece of the intermediate, K streamed through LDS in tiles of 64
//      (transposed product, a lane owns a token row, as in the other GEMMs of this library),
//   2. applies bias + activation and leaves the piece in LDS in fp16 (the reference rounds the
//      intermediate to fp16 as well, gemm_gemm.py:152), laid out as the K-contiguous operand of
//   3. the second product: its contribution Y[64, H] += piece[64,128] @ W2t[:, chunk]^T, W2t
//      streamed in tiles of 128 output columns, added to an fp32 workspace with atomic adds
//      (this product is formed non-transposed: a lane owns an output column, so one atomic
//      instruction covers two rows of 32 consecutive floats);
//   4. the workgroup that arrives last at a row block (a counter per row block; nobody waits)
//      converts the sums to fp16 (+ b2), writes Y and returns the workspace to zeros.
// Meant for small token counts (M <= ~1024), where two separate GEMM launches run at the latency
// of their K loops on a few dozen workgroups: the chunk split gives M/64 * F/128 workgroups (192
// at M 512, F 3072) and the second product a K of 128 per workgroup.
// MEASURED (MI355X, M 512, K 768, F 3072, H 768): 67 us against 31 us for the two launches it
// replaces (9 + 22 us), so no caller of this library selects it by default.  About 40 us remain
// without the atomic adds (one workgroup of four waves per compute unit, a load of 24-32 KB
// awaited at every step: the K loops run at the load latency) and the 9.4 M fp32 atomic adds
// (24 partial results per output element) cost the other 27 us, which no pipelining of the loops
// removes.
// Fewer partial results mean fewer workgroups (F / chunk of them per row block), each streaming
// more of the 9.4 MB of weights through one compute unit; at this M the split that keeps the
// intermediate on chip and the parallelism the chip needs exclude each other.
// fp32 atomic accumulation makes the summation order of the F/128 contributions vary from run
// to run (differences far below the fp16 output grid).
#include <algorithm>
#include "stof_common.h"

namespace {

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(1))) const void gptr_t;

__device__ __forceinline__ floatx16 mfma32(half8_t a, half8_t b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// chunk c (16 B) of a 128-byte tile row r is stored at chunk position c ^ swz(r)
__device__ __forceinline__ int swz(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }
__device__ __forceinline__ half8_t lds_frag(const lds_byte* tile, int byte_off) {
  return *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(tile + byte_off);
}
__device__ __forceinline__ void dma16(const half_t* src, lds_byte* dst) {
  __builtin_amdgcn_global_load_lds((gptr_t*)src, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
}

struct ChainParams {
  const half_t* X; const half_t* W1; const half_t* b1; const half_t* W2; const half_t* b2; half_t* Y;
  float* ws; int* counters;
  int M, K, F, H; int ldx, ldy;
  int tiles_m, chunks;
};

constexpr int kRows = 64;      // tokens per workgroup
constexpr int kChunk = 128;    // intermediate features per workgroup
constexpr int kKT = 64;        // K per tile of the first product
constexpr int kNT = 128;       // output columns per tile of the second product
constexpr int kPanel = 64 * 128;   // bytes of a 64-row panel of 64 halves

template <int ACT>
__global__ __launch_bounds__(256) void ffn_chain_kernel(const ChainParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char x_lds0[kPanel];        // X tile: 64 tokens x 64 k
  __shared__ __attribute__((aligned(1024))) unsigned char x_lds1[kPanel];
  __shared__ __attribute__((aligned(1024))) unsigned char w1_lds0[2 * kPanel];   // W1 tile: 128 features x 64 k
  __shared__ __attribute__((aligned(1024))) unsigned char w1_lds1[2 * kPanel];
  __shared__ __attribute__((aligned(1024))) unsigned char h_lds[2 * kPanel];     // the piece: two panels of 64 tokens x 64 features
  __shared__ __attribute__((aligned(1024))) unsigned char w2_lds0[4 * kPanel];   // W2 tile: two panels of 128 columns x 64 features
  __shared__ __attribute__((aligned(1024))) unsigned char w2_lds1[4 * kPanel];
  __shared__ int s_last;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31, g = lane >> 5;
  const int wt = wave & 1, wf = wave >> 1;   // token half (32), feature / column half (64)

  // consecutive workgroups share the chunk (the same rows of W1t and columns of W2t) and walk the row blocks
  const int mt = blockIdx.x % p.tiles_m;
  const int fc = blockIdx.x / p.tiles_m;
  const int m0 = mt * kRows, f0 = fc * kChunk;

  // ---- loads.  One instruction = 8 rows of 128 B.
  const int lrow = lane >> 3;
  const half_t* x_src[2]; const half_t* w1_src[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int trow = 8 * (2 * wave + i) + lrow;
    x_src[i] = p.X + (int64_t)min(m0 + trow, p.M - 1) * p.ldx + 8 * ((lane & 7) ^ swz(trow));   // rows past the edge re-read the last row
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int trow = 8 * (4 * wave + i) + lrow;
    w1_src[i] = p.W1 + (int64_t)(f0 + trow) * p.K + 8 * ((lane & 7) ^ swz(trow));
  }
  auto issue1 = [&](int kt, lds_byte* xd, lds_byte* wd) {
#pragma unroll
    for (int i = 0; i < 2; ++i) dma16(x_src[i] + kt * kKT, xd + (2 * wave + i) * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(w1_src[i] + kt * kKT, wd + (4 * wave + i) * 1024);
  };
  // W2 tile nt: rows = output columns 128 nt .. 128 nt + 127, two panels of 64 features of the chunk
  const half_t* w2_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int trow = 8 * (4 * wave + i) + lrow;
    w2_src[i] = p.W2 + (int64_t)trow * p.F + f0 + 8 * ((lane & 7) ^ swz(trow));
  }
  auto issue2 = [&](int nt, lds_byte* wd) {
#pragma unroll
    for (int kp = 0; kp < 2; ++kp)
#pragma unroll
      for (int i = 0; i < 4; ++i) dma16(w2_src[i] + (int64_t)nt * kNT * p.F + 64 * kp, wd + kp * 2 * kPanel + (4 * wave + i) * 1024);
  };
  // fragment read offsets: row j32 of a 32-row group, chunk 2*ks + g
  int rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) rd[ks] = j32 * 128 + (((2 * ks + g) ^ swz(j32)) << 4);

  // ---- 1. piece^T = W1t[chunk] . X^T : acc1[ni][r] = piece[32 wt + j32][64 wf + 32 ni + 8 (r / 4) + 4 g + r % 4]
  floatx16 acc1[2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[ni][r] = 0.f;
  auto compute1 = [&](const lds_byte* xt, const lds_byte* wtile) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const half8_t xa = lds_frag(xt, (32 * wt) * 128 + rd[ks]);
      half8_t wb[2];
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) wb[ni] = lds_frag(wtile, (64 * wf + 32 * ni) * 128 + rd[ks]);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) acc1[ni] = mfma32(wb[ni], xa, acc1[ni]);
    }
  };
  const int nk = p.K / kKT;
  issue1(0, (lds_byte*)x_lds0, (lds_byte*)w1_lds0);
  for (int kt = 0; kt < nk; kt += 2) {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's share of tile kt landed
    __syncthreads();
    if (kt + 1 < nk) issue1(kt + 1, (lds_byte*)x_lds1, (lds_byte*)w1_lds1);
    compute1((const lds_byte*)x_lds0, (const lds_byte*)w1_lds0);
    if (kt + 1 < nk) {   // (no early exit from the loop: a second exit makes the compiler copy the accumulators)
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (kt + 2 < nk) issue1(kt + 2, (lds_byte*)x_lds0, (lds_byte*)w1_lds0);
      compute1((const lds_byte*)x_lds1, (const lds_byte*)w1_lds1);
    }
  }

  // ---- 2. bias + activation, fp16, into LDS as the K-contiguous operand of the second product.
  // The first two W2 tiles are requested first, so they arrive under the activation arithmetic.
  const int n_tiles = p.H / kNT;
  issue2(0, (lds_byte*)w2_lds0);
  if (n_tiles > 1) issue2(1, (lds_byte*)w2_lds1);
  {
    const int row = 32 * wt + j32;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        half4_t bv = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        if (p.b1) bv = *reinterpret_cast<const half4_t*>(p.b1 + f0 + 64 * wf + 32 * ni + 8 * q4 + 4 * g);
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (half_t)activate<ACT>(acc1[ni][4 * q4 + e] + (float)bv[e]);
        // panel wf, row `row`, features 32 ni + 8 q4 + 4 g .. + 3 of the panel: chunk 4 ni + q4, half g
        *reinterpret_cast<__attribute__((address_space(3))) half4_t*>((lds_byte*)h_lds + wf * kPanel + row * 128 + (((4 * ni + q4) ^ swz(row)) << 4) + 8 * g) = o;
      }
  }

  // ---- 3. Y[tokens, columns] += piece . W2t[columns, chunk]^T, non-transposed:
  // acc2[ni][r] = Y[32 wt + 8 (r / 4) + 4 g + r % 4][128 nt + 64 wf + 32 ni + j32]
  floatx16 acc2[2];
  auto compute2 = [&](const lds_byte* w2t) {
#pragma unroll
    for (int kp = 0; kp < 2; ++kp)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const half8_t ha = lds_frag((const lds_byte*)h_lds + kp * kPanel, (32 * wt) * 128 + rd[ks]);
        half8_t wb[2];
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) wb[ni] = lds_frag(w2t + kp * 2 * kPanel, (64 * wf + 32 * ni) * 128 + rd[ks]);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) acc2[ni] = mfma32(ha, wb[ni], acc2[ni]);
      }
  };
  auto add_out = [&](int nt) {
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      float* col = p.ws + 128 * nt + 64 * wf + 32 * ni + j32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + 32 * wt + 8 * (r >> 2) + 4 * g + (r & 3);
        if (m < p.M) unsafeAtomicAdd(col + (int64_t)m * p.H, acc2[ni][r]);
      }
    }
  };
  for (int nt = 0; nt < n_tiles; nt += 2) {
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[ni][r] = 0.f;
    __builtin_amdgcn_s_waitcnt(0x0F70);   // tile nt landed
    __syncthreads();                      // (first pass: the piece is complete in LDS; later: everyone is done with tile nt - 1)
    if (nt >= 1 && nt + 1 < n_tiles) issue2(nt + 1, (lds_byte*)w2_lds1);
    compute2((const lds_byte*)w2_lds0);
    add_out(nt);
    if (nt + 1 < n_tiles) {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[ni][r] = 0.f;
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (nt + 2 < n_tiles) issue2(nt + 2, (lds_byte*)w2_lds0);
      compute2((const lds_byte*)w2_lds1);
      add_out(nt + 1);
    }
  }

  // ---- 4. the last workgroup of this row block converts the sums
  // The sums live in device-scope atomics, which do not stay in this XCD's L2, so no cache
  // write-back is needed before the counter moves (a fence of device scope would write back the
  // whole L2 once per workgroup: measured 20+ us per launch).  Each thread waits for its own
  // atomic adds to be acknowledged, the barrier collects the workgroup, then the counter moves.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  __syncthreads();
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(p.counters + mt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (prev == p.chunks - 1);
  }
  __syncthreads();
  if (!s_last) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // the reader drops what its caches hold of the sums
  const int quads = p.H / 4;
  for (int idx = threadIdx.x; idx < kRows * quads; idx += 256) {
    const int r = idx / quads, c = 4 * (idx % quads);
    const int m = m0 + r;
    if (m >= p.M) break;
    float* src = p.ws + (int64_t)m * p.H + c;
    const floatx4 v4 = *reinterpret_cast<const floatx4*>(src);
    half4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (half_t)(v4[e] + (p.b2 ? (float)p.b2[c + e] : 0.f));
    *reinterpret_cast<half4_t*>(p.Y + (int64_t)m * p.ldy + c) = o;
    *reinterpret_cast<floatx4*>(src) = floatx4{0.f, 0.f, 0.f, 0.f};   // the workspace goes back to zeros for the next call
  }
  if (threadIdx.x == 0) p.counters[mt] = 0;
}

int64_t counters_offset(int64_t M, int64_t H) { return ((M * H * 4 + 255) / 256) * 256; }

}  // namespace

extern "C" int64_t stof_gemm_act_gemm_workspace_bytes(int64_t M, int64_t H) {
  if (M <= 0 || H <= 0) return 0;
  return counters_offset(M, H) + ((M + kRows - 1) / kRows) * 4;
}

extern "C" int stof_gemm_act_gemm(const void* X, const void* W1t, const void* b1, const void* W2t, const void* b2,
                                  void* Y, int64_t M, int64_t K, int64_t F, int64_t H, int64_t ldx, int64_t ldy,
                                  int act, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!X || !W1t || !W2t || !Y || !workspace) return STOF_ERR_NULL_POINTER;
  if (M <= 0 || K <= 0 || F <= 0 || H <= 0 || K % kKT != 0 || F % kChunk != 0 || H % kNT != 0 || ldx < K || ldy < H)
    return STOF_ERR_BAD_SHAPE;
  if (M > (1 << 24) || K > (1 << 24) || F > (1 << 24) || H > (1 << 24)) return STOF_ERR_BAD_SHAPE;
  if (!stof_aligned16(X) || !stof_aligned16(W1t) || !stof_aligned16(W2t) || ((uintptr_t)Y & 7) ||
      ((uintptr_t)b1 & 7) || ((uintptr_t)b2 & 7) || ((uintptr_t)workspace & 15) || ldx % 8 != 0 || ldy % 4 != 0)
    return STOF_ERR_MISALIGNED;
  if (workspace_bytes < stof_gemm_act_gemm_workspace_bytes(M, H)) return STOF_ERR_BAD_SHAPE;
  ChainParams p;
  p.X = (const half_t*)X; p.W1 = (const half_t*)W1t; p.b1 = (const half_t*)b1; p.W2 = (const half_t*)W2t;
  p.b2 = (const half_t*)b2; p.Y = (half_t*)Y;
  p.ws = (float*)workspace;
  p.counters = reinterpret_cast<int*>(reinterpret_cast<char*>(workspace) + counters_offset(M, H));
  p.M = (int)M; p.K = (int)K; p.F = (int)F; p.H = (int)H; p.ldx = (int)ldx; p.ldy = (int)ldy;
  p.tiles_m = (int)((M + kRows - 1) / kRows); p.chunks = (int)(F / kChunk);
  const int64_t groups = (int64_t)p.tiles_m * p.chunks;
  if (groups > (1 << 30)) return STOF_ERR_BAD_SHAPE;
  const dim3 grid((unsigned)groups), block(256);
  hipStream_t st = (hipStream_t)stream;
  switch (act) {
    case STOF_ACT_NONE: hipLaunchKernelGGL(ffn_chain_kernel<STOF_ACT_NONE>, grid, block, 0, st, p); break;
    case STOF_ACT_GELU_ERF: hipLaunchKernelGGL(ffn_chain_kernel<STOF_ACT_GELU_ERF>, grid, block, 0, st, p); break;
    case STOF_ACT_GELU_TANH: hipLaunchKernelGGL(ffn_chain_kernel<STOF_ACT_GELU_TANH>, grid, block, 0, st, p); break;
    case STOF_ACT_RELU: hipLaunchKernelGGL(ffn_chain_kernel<STOF_ACT_RELU>, grid, block, 0, st, p); break;
    default: return STOF_ERR_UNSUPPORTED;
  }
  return stof_check_launch();
}
