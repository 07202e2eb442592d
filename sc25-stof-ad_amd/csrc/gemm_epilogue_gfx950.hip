// Fused encoder GEMMs for gfx950 (MI355X):
//   stof_gemm_bias_act, stof_gemm_bias_act_splitk       C = act(A @ W^T + bias)       (bias / GELU / ReLU epilogue)
//   stof_gemm_bias_res_ln, stof_gemm_bias_res_ln_cluster  C = LN(A @ W^T + bias + residual) * g + b   (LayerNorm epilogue)
//
// They replace the reference's Triton templates (src/triton_template/gemm_gemm.py:99-150,
// src/triton_template/gemm_add_layernorm.py:78-123).  Common design:
//
//  * both operands are K-contiguous (A [M,K], Wt [N,K]) and travel L2 -> LDS with
//    direct-to-LDS loads, double buffered, one barrier per K tile; LDS tiles are unpadded
//    rows of 128 B (64 halves) with a 16-byte-chunk XOR swizzle, so the 16-byte fragment
//    reads of 16 consecutive rows hit distinct banks;
//  * the product is formed TRANSPOSED, C^T = Wt . A^T, with v_mfma_f32_32x32x16_f16: the
//    weights are the A operand, the activations the B operand.  In the accumulator layout
//    a lane then owns ONE token row (lane & 31) and its registers run along the feature
//    dimension in groups of four consecutive columns.  Bias, activation, residual and the
//    LayerNorm statistics become per-lane register loops, and stores are 8-byte vectors;
//  * the LayerNorm kernels keep the pre-normalisation tensor on chip: either one workgroup
//    (8 waves) owns the full row of N features, each wave a slice of N/8 columns, with mean
//    and variance reduced in registers, across the lane pair with v_permlane32_swap and across
//    the 8 waves through 2 KB of LDS; or the N / 128 workgroups of a block of 128 token rows
//    each own a 128 x 128 tile and exchange per-row statistics through a small workspace.
#include "stof_common.h"

namespace {

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(1))) const void gptr_t;

__device__ __forceinline__ float pair_sum(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}
// chunk c (16 B) of tile row r is stored at chunk position c ^ swz(r)
__device__ __forceinline__ int swz(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

__device__ __forceinline__ half8_t lds_frag(const lds_byte* tile, int byte_off) {
  return *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(tile + byte_off);
}
__device__ __forceinline__ void dma16(const half_t* src, lds_byte* dst) {
  __builtin_amdgcn_global_load_lds((gptr_t*)src, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
}
// The operand tiles of the K loops are addressed through buffer resources: the tile's first row as
// a wave-uniform base in scalar registers (set up once per workgroup), the lane's place inside the
// tile as a 32-bit byte offset computed once, the position along K as a scalar offset - no 64-bit
// vector add per load instruction.  (Extent 2^32 - 1: every address is in range by construction,
// rows past the edge re-read the last row.)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const half_t* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(base), 0, -1, 0x00020000);
}
__device__ __forceinline__ void dma16b(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t k_off, lds_byte* dst) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, lane_off, k_off, 0, 0);
}

struct GemmParams {
  const half_t* A; const half_t* W; const half_t* bias; half_t* C;
  int M, N, K; int lda, ldc;
  int tiles_m, tiles_n;
  // split-K launches only: workgroup (tile, z) multiplies k-tiles [z * nk_split, (z + 1) * nk_split)
  float* partials; int* counters; int splits; int nk_split;
};

// Workgroup index -> output tile.  Workgroups go round-robin to the 8 XCDs, each with an L2 of
// its own, and about 64 of them run on an XCD at a time.  XCD x = index % 8 owns the token tiles
// tm = 8 q + x and takes its tiles in bands of kRasterRows values of q, feature tile after feature
// tile inside a band: the 64 workgroups in flight on an XCD then cover 8 token tiles x 8 feature
// tiles and bring 8 + 8 operand tiles through its L2 instead of 64 + 1 (token tile after token
// tile for one feature tile re-read the activations once per feature tile from memory:
// 65536 x 3072 x 768 470 us = 660 TFLOP/s where 8192 rows reach 840).
// The grid is 8 * ceil(tiles_m / 8) * tiles_n; false = padding of the last token tiles.
constexpr int kRasterRows = 8;
__device__ __forceinline__ bool raster_tile(int index, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int x = index & 7, i = index >> 3;
  const int rows_x = (tiles_m + 7) >> 3;
  const int band = i / (kRasterRows * tiles_n), r = i - band * (kRasterRows * tiles_n);
  const int first = band * kRasterRows;
  const int rows = min(kRasterRows, rows_x - first);
  tn = r / rows;
  tm = 8 * (first + r - tn * rows) + x;
  return tm < tiles_m;
}
inline unsigned raster_grid(int tiles_m, int tiles_n) { return 8u * (unsigned)((tiles_m + 7) / 8) * (unsigned)tiles_n; }

// Epilogue of the bias / activation GEMMs for one wave: acc[ni][mi][r] is
// C[m_base + 32 mi + j32][n_base + 32 ni + 8 (r / 4) + 4 g + r % 4].  In this layout a store
// instruction would write 16 B into each of 32 rows, 32 partial cache lines per instruction
// (measured on 8192 x 3072 outputs: 2.9 TB/s, the stores alone 17 us).  Each block of 32 tokens x 64
// features therefore goes through 4 KB of LDS of the wave's own (the operand tiles are free
// after the last k-step; rows of 128 B with the 16-byte chunk index XOR-ed by the row, so the
// row-wise reads are conflict-free) and leaves as 4 stores of 8 full 128-byte lines each.
template <int ACT, int MT, bool BF = false>
__device__ __forceinline__ void store_wave_block(const GemmParams& p, const floatx16 (&acc)[2][MT], lds_byte* stage,
                                                 int m_base, int n_base, int lane) {
  const int j32 = lane & 31, g = lane >> 5;
  // the wave's block of C as a buffer: base = its first element, 32-bit byte offsets per lane (ldc < 2^23, host-checked)
  const __amdgpu_buffer_rsrc_t c_rsrc = stof_wave_rsrc(p.C + (int64_t)m_base * p.ldc + n_base);
  half4_t bv[2][4];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int n = n_base + 32 * ni + 8 * q4 + 4 * g;
      bv[ni][q4] = half4_t{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
      if (p.bias && n < p.N) bv[ni][q4] = *reinterpret_cast<const half4_t*>(p.bias + n);   // N % 8 == 0: a group of 4 is inside or outside as a whole
    }
#pragma unroll
  for (int mi = 0; mi < MT; ++mi) {
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const half_t be = bv[ni][q4][e];
          o[e] = to_elem<BF>(activate<ACT>(acc[ni][mi][4 * q4 + e] + from_elem<BF>(be)));
        }
        *reinterpret_cast<__attribute__((address_space(3))) half4_t*>(stage + j32 * 128 + (((4 * ni + q4) ^ (j32 & 7)) << 4) + 8 * g) = o;
      }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 8 * i + (lane >> 3), c = lane & 7;
      const half8_t o = *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(stage + t * 128 + ((c ^ (t & 7)) << 4));
      const int m = m_base + 32 * mi + t, n = n_base + 8 * c;
      // (written through the XCD's cache, so the tile is on its way to memory while the kernel runs and
      // not part of the end-of-kernel write-back the next launch waits for: a BERT-large layer of five
      // launches at 8192 tokens 282 -> 269 us, BERT-base 185 -> 184)
      if (m < p.M && n < p.N) stof_store16_through(c_rsrc, (uint32_t)(32 * mi + t) * (uint32_t)(p.ldc * 2) + 16 * c, o);
    }
  }
}

// Split-K hand-over for one wave (launches with p.splits > 1: the grid is `splits` copies of the
// tile grid, copy z has multiplied the z-th range of k-tiles).  The wave hands its partial sums
// (acc, 32 * MT floats per lane) to the wave of the same place in the split that finishes last:
// 8-byte device-scope stores (written through to memory, 512 contiguous bytes per instruction), a
// wait until they are acknowledged, then one count on the (tile, wave) counter.  The wave that
// counts last adds the partial sums in the order of z - its own from registers - so the result
// does not depend on which split came last, puts the counter back to zero for the next launch and
// returns true with the total in acc; the others return false and are done.
template <int MT>
__device__ __forceinline__ bool splitk_handover(const GemmParams& p, floatx16 (&acc)[2][MT], int64_t tile, int z, int wave, int lane) {
  typedef unsigned long long u64;
  constexpr int kSlot = 1024 * MT;   // 8-byte words per (tile, split, wave)
  u64* mine = reinterpret_cast<u64*>(p.partials) + ((tile * p.splits + z) * 4 + wave) * kSlot + lane;
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        // (through scalar copies: a bit cast applied directly to a vector element reads element 0)
        const float lo = acc[ni][mi][r], hi = acc[ni][mi][r + 1];
        const u64 v = ((u64)__builtin_bit_cast(unsigned, hi) << 32) | __builtin_bit_cast(unsigned, lo);
        __hip_atomic_store(mine + ((ni * MT + mi) * 8 + (r >> 1)) * 64, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
  // (relaxed atomics to different addresses are not ordered for the compiler: the empty asm
  // statements keep the stores above the wait, the count below it and the reads below the count)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  asm volatile("" ::: "memory");
  int* counter = p.counters + tile * 4 + wave;
  int before = 0;
  if (lane == 0) before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  before = __builtin_amdgcn_readfirstlane(before);
  asm volatile("" ::: "memory");
  if (before != p.splits - 1) return false;
  floatx16 sum[2][MT];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum[ni][mi][r] = 0.f;
  const u64* slot0 = reinterpret_cast<const u64*>(p.partials) + ((tile * p.splits) * 4 + wave) * kSlot + lane;
  for (int zz = 0; zz < p.splits; ++zz) {
    if (zz == z) {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int mi = 0; mi < MT; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) sum[ni][mi][r] += acc[ni][mi][r];
    } else {
      const u64* src = slot0 + (int64_t)zz * 4 * kSlot;
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int mi = 0; mi < MT; ++mi)
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const u64 v = __hip_atomic_load(src + ((ni * MT + mi) * 8 + (r >> 1)) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum[ni][mi][r] += __builtin_bit_cast(float, (unsigned)(v & 0xffffffffull));
            sum[ni][mi][r + 1] += __builtin_bit_cast(float, (unsigned)(v >> 32));
          }
    }
  }
  if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < MT; ++mi) acc[ni][mi] = sum[ni][mi];
  return true;
}

// ------------------------------------------------------------------------------------------
// C[M,N] = act(A[M,K] @ Wt[N,K]^T + bias[N]);  tile 128 (tokens) x 128 (features) x 64 (K),
// 4 waves as 2 x 2, each 64 tokens x 64 features = 2 x 2 MFMA tiles.
// ------------------------------------------------------------------------------------------

constexpr int kGT = 128;            // tile edge (tokens and features)
constexpr int kGK = 64;             // K per tile
constexpr int kGTile = kGT * kGK * 2;   // bytes per operand tile (16 KB)

template <int ACT, bool SK = false, bool BF = false>
__global__ __launch_bounds__(256) void gemm_bias_act_kernel(const GemmParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds0[kGTile];
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds1[kGTile];
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds0[kGTile];
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds1[kGTile];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31, g = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;

  // split-K: the grid is `splits` copies of the tile grid, copy z takes the z-th range of k-tiles
  const int tile_grid = (int)(8u * (unsigned)((p.tiles_m + 7) / 8) * (unsigned)p.tiles_n);
  const int z = SK ? (int)blockIdx.x / tile_grid : 0;
  int tm, tn;
  if (!raster_tile((int)blockIdx.x - z * tile_grid, p.tiles_m, p.tiles_n, tm, tn)) return;
  const int m0 = tm * kGT, n0 = tn * kGT;
  const int kt_first = SK ? z * p.nk_split : 0;

  // DMA: 16 instructions of 8 rows per operand tile; wave w issues 4w..4w+3.
  uint32_t a_off[4], w_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int trow = 8 * (4 * wave + i) + (lane >> 3);
    const int chunk = (lane & 7) ^ swz(trow);
    a_off[i] = (uint32_t)min(trow, p.M - 1 - m0) * (uint32_t)(p.lda * 2) + 16 * chunk;   // rows past the edge re-read the last row
    w_off[i] = (uint32_t)min(trow, p.N - 1 - n0) * (uint32_t)(p.K * 2) + 16 * chunk;
  }
  const __amdgpu_buffer_rsrc_t a_rs = tile_rsrc(p.A + (int64_t)m0 * p.lda), w_rs = tile_rsrc(p.W + (int64_t)n0 * p.K);
  auto issue = [&](int kt, lds_byte* ad, lds_byte* wd) {
    const uint32_t koff = (uint32_t)(kt_first + kt) * (kGK * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16b(a_rs, a_off[i], koff, ad + (4 * wave + i) * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16b(w_rs, w_off[i], koff, wd + (4 * wave + i) * 1024);
  };
  // fragment read offsets: row (32*t + j32), chunk 2*ks + g
  int rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) rd[ks] = j32 * 128 + (((2 * ks + g) ^ swz(j32)) << 4);

  floatx16 acc[2][2];   // [feature tile ni][token tile mi]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Fragments of k-step ks + 1 are requested before the MFMAs of k-step ks are issued (two sets of
  // fragment registers), so the LDS latency of a k-step hides behind the previous one's products.
  auto compute = [&](const lds_byte* at, const lds_byte* wt) {
    half8_t xa[2][2], wb[2][2];
    auto fetch = [&](int ks, int set) {
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) xa[set][mi] = lds_frag(at, (64 * wm + 32 * mi) * 128 + rd[ks]);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) wb[set][ni] = lds_frag(wt, (64 * wn + 32 * ni) * 128 + rd[ks]);
    };
    fetch(0, 0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) fetch(ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) acc[ni][mi] = mfma32<BF>(wb[ks & 1][ni], xa[ks & 1][mi], acc[ni][mi]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nk = SK ? min(p.nk_split, p.K / kGK - kt_first) : p.K / kGK;
  issue(0, (lds_byte*)a_lds0, (lds_byte*)w_lds0);
  for (int kt = 0; kt < nk; kt += 2) {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's share of tile kt landed
    __syncthreads();
    if (kt + 1 < nk) issue(kt + 1, (lds_byte*)a_lds1, (lds_byte*)w_lds1);
    compute((const lds_byte*)a_lds0, (const lds_byte*)w_lds0);
    if (kt + 1 < nk) {   // (no early exit from the loop: a second exit makes the compiler copy the accumulators)
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (kt + 2 < nk) issue(kt + 2, (lds_byte*)a_lds0, (lds_byte*)w_lds0);
      compute((const lds_byte*)a_lds1, (const lds_byte*)w_lds1);
    }
  }

  __syncthreads();   // every wave is done with the operand tiles
  if constexpr (SK) {
    if (!splitk_handover<2>(p, acc, (int64_t)tm * p.tiles_n + tn, z, wave, lane)) return;
  }
  store_wave_block<ACT, 2, BF>(p, acc, (lds_byte*)a_lds0 + wave * 4096, m0 + 64 * wm, n0 + 64 * wn, lane);
}

// ------------------------------------------------------------------------------------------
// Ring form of the same GEMM for small token counts: tile 64 (tokens) x 128 (features) x KT (K),
// 4 waves as 2 x 2, each 32 tokens x 64 features = 2 MFMA tiles; four times the workgroups of the
// 128 x 128 form.  The K loop is a ring of NS stages filled by direct-to-LDS loads (NS - 1 tiles
// in flight per workgroup) and is software pipelined inside the wave: the form for token counts
// that give the 128 x 128 form less than one workgroup per two compute units, where the K loop
// of each workgroup runs at the latency of its loads.  Launched with KT = 64, NS = 3 (72 KB of
// LDS, two workgroups per compute unit, 48 KB in flight per workgroup, one barrier per 64 of K);
// KT = 32, NS = 4 (36 KB in flight, a barrier per 32 of K) was the first version: 512 tokens,
// N 768, K 3072 22.1 -> 17.9 us, N 1024, K 4096 27.6 -> 22.4, 2048 x 768 x 3072 22.6 -> 18.8;
// K 768 unchanged (8 us, the pace of the launches).  NS = 4 with KT = 64 measures like NS = 3,
// NS = 2 is 50 % slower.  With SK the K dimension is split over several workgroups per tile as well.
// (The same structure with 256-token tiles and three stages - 0.75 KB of LDS reads per MFMA
// instead of 1 KB - was the form for large grids until the 128 x 128 form got buffer-resource
// loads and the banded tile order; it is no longer part of the library.)
// ------------------------------------------------------------------------------------------
constexpr int kWFeat = 128;
constexpr int kSmallKT = 64;          // K per tile of the ring form as it is launched

// 64-byte rows: chunk c of row r sits at position c ^ ((r >> 2) & 3); 16 rows fill 1 KB.
__device__ __forceinline__ int swz4(int row) { return (row >> 2) & 3; }

// s_waitcnt immediate that waits for the vector-memory counter only (lgkmcnt 15, expcnt 7)
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

template <int ACT, int NS, bool SK = false, int KT = kSmallKT, bool BF = false>
__global__ __launch_bounds__(256, 2) void gemm_bias_act_ring_kernel(const GemmParams p) {
  static_assert(KT == 32 || KT == 64, "K per tile");
  constexpr int kK = KT;
  constexpr int kTok = 64;                // tokens per workgroup: two waves of 32
  constexpr int kPitch = kK * 2;          // bytes per tile row
  constexpr int kRowsPI = 1024 / kPitch;  // tile rows per load instruction (1 KB)
  constexpr int kAI = kTok / kRowsPI / 4, kWI = kWFeat / kRowsPI / 4;   // load instructions per wave: A tile, W tile
  constexpr int kLoads = kAI + kWI;       // per wave per tile
  constexpr int kKS = kK / 16;            // k-steps (MFMA depth 16) per tile
  constexpr int kATile = kTok * kPitch, kWTile = kWFeat * kPitch;   // 4 / 8 KB, 8 / 16 KB
  // Ring of NS stages: NS tiles are in flight or in use at any time, so a tile has NS - 1 tile
  // times to arrive.  (The fragment reads below are asm, so the compiler does not order them
  // against the direct-to-LDS loads and one array per operand is enough.)
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds[NS * kATile];
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds[NS * kWTile];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31, g = lane >> 5;
  const int wf = wave >> 1, wt = wave & 1;   // feature half (64), token half (32)

  // split-K: the grid is `splits` copies of the tile grid, copy z takes the z-th range of k-tiles
  const int tile_grid = (int)(8u * (unsigned)((p.tiles_m + 7) / 8) * (unsigned)p.tiles_n);
  const int z = SK ? (int)blockIdx.x / tile_grid : 0;
  int tm, tn;
  if (!raster_tile((int)blockIdx.x - z * tile_grid, p.tiles_m, p.tiles_n, tm, tn)) return;
  const int m0 = tm * kTok, n0 = tn * kWFeat;
  const int kt_first = SK ? z * p.nk_split : 0;

  // Loads: one instruction = 1 KB = kRowsPI tile rows.  Rows past the edge re-read the last row.
  // 16-byte chunk c of tile row r sits at chunk position c ^ sw(r) (sw: 2 bits for 64-byte rows,
  // 3 bits for 128-byte rows), so the fragment reads of 32 consecutive rows spread over the banks.
  // Plain global addresses: the K loop runs at the latency of its loads, and the buffer-resource
  // form that the 128 x 128 kernel gains from measured 10-25 % slower here (512 x 3072 x 768:
  // 11.4 vs 9.1 us).
  auto sw = [](int row) { return KT == 32 ? swz4(row) : swz(row); };
  constexpr int kChunks = kPitch / 16;
  const int drow = lane / kChunks, dchunk = lane % kChunks;
  uint32_t a_off[kAI], w_off[kWI];
#pragma unroll
  for (int i = 0; i < kAI; ++i) {
    const int trow = kRowsPI * (kAI * wave + i) + drow;
    a_off[i] = (uint32_t)min(trow, p.M - 1 - m0) * (uint32_t)(p.lda * 2) + 16 * (dchunk ^ sw(trow));
  }
#pragma unroll
  for (int i = 0; i < kWI; ++i) {
    const int trow = kRowsPI * (kWI * wave + i) + drow;
    w_off[i] = (uint32_t)min(trow, p.N - 1 - n0) * (uint32_t)(p.K * 2) + 16 * (dchunk ^ sw(trow));
  }
  const char* a_first = reinterpret_cast<const char*>(p.A + (int64_t)m0 * p.lda);
  const char* w_first = reinterpret_cast<const char*>(p.W + (int64_t)n0 * p.K);
  auto issue = [&](int kt, int stage) {
    const uint32_t koff = (uint32_t)(kt_first + kt) * kPitch;
    lds_byte* ad = (lds_byte*)a_lds + stage * kATile;
    lds_byte* wd = (lds_byte*)w_lds + stage * kWTile;
#pragma unroll
    for (int i = 0; i < kAI; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t*)(a_first + koff + a_off[i]), (__attribute__((address_space(3))) void*)(ad + (kAI * wave + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < kWI; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t*)(w_first + koff + w_off[i]), (__attribute__((address_space(3))) void*)(wd + (kWI * wave + i) * 1024), 16, 0, 0);
  };
  // fragment read: row (32*t + j32), chunk 2*ks + g
  int rd[kKS];
#pragma unroll
  for (int ks = 0; ks < kKS; ++ks) rd[ks] = j32 * kPitch + (((2 * ks + g) ^ sw(j32)) << 4);

  floatx16 acc[2][1];   // [feature tile ni][token tile]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][0][r] = 0.f;

  // Fragment reads are written as asm: the compiler orders LDS reads it can see after every
  // direct-to-LDS load it cannot prove disjoint, which drains the ring.  The ring's own
  // counter waits cover that dependency; the LDS counter is waited on by hand (lds_wait).
  auto frags = [&](uint32_t wa, uint32_t aa, half8_t (&wbk)[2], half8_t& xak) {
    asm volatile(
        "ds_read_b128 %0, %3\n\tds_read_b128 %1, %3 offset:%5\n\t"
        "ds_read_b128 %2, %4"
        : "=&v"(wbk[0]), "=&v"(wbk[1]), "=&v"(xak)
        : "v"(wa), "v"(aa), "n"(32 * kPitch));
  };
  // Wait for the fragment reads of one set: all reads (newer_in_flight false) or all but the
  // 3 reads of the set requested last.  The wait is an asm statement that names the
  // fragments it covers as read-write operands, so every use of them depends on it and neither
  // the scheduler nor the register allocator can move a use (or a copy) above the wait.  The LDS
  // counter is shared with scalar loads, which return out of order: an outstanding one can only
  // make this wait longer, never shorter, because LDS reads return in order among themselves.
  auto lds_wait = [&](bool newer_in_flight, half8_t (&wbk)[2], half8_t& xak) {
    __builtin_amdgcn_sched_barrier(0);   // (keeps the software pipeline in the order written)
    if (newer_in_flight) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(wbk[0]), "+v"(wbk[1]), "+v"(xak));
    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wbk[0]), "+v"(wbk[1]), "+v"(xak));
    __builtin_amdgcn_sched_barrier(0);
  };
  auto mfmas = [&](const half8_t (&wbk)[2], const half8_t& xak) {
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) acc[ni][0] = mfma32<BF>(wbk[ni], xak, acc[ni][0]);
  };
  auto wg_barrier = [&]() {
    // bare barrier: the fences of __syncthreads() would drain the loads that must stay in flight
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  const uint32_t w_rd = (uint32_t)(uintptr_t)(lds_byte*)w_lds + (uint32_t)(64 * wf) * kPitch;
  const uint32_t a_rd = (uint32_t)(uintptr_t)(lds_byte*)a_lds + (uint32_t)(32 * wt) * kPitch;
  half8_t xa[2], wb[2][2];   // two sets of fragments: k-step ks uses set ks & 1

  const int nk = SK ? min(p.nk_split, p.K / kK - kt_first) : p.K / kK;
#pragma unroll
  for (int s0 = 0; s0 < NS; ++s0)
    if (s0 < nk) issue(s0, s0);
  if (nk >= NS) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads * (NS - 1)));   // tile 0 landed
  else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  wg_barrier();
  frags(w_rd + rd[0], a_rd + rd[0], wb[0], xa[0]);
  // Tile t: the reads of k-step ks + 1 go out before the MFMAs of k-step ks; during the last
  // k-step tile t+1 is awaited, the barrier lets tile t's stage be refilled with tile t+NS, and
  // the first fragments of tile t+1 are read while the MFMAs of that last k-step execute.
  int cs = 0;   // stage of tile t
  for (int t = 0; t < nk; ++t) {
    const int ns = (cs + 1 == NS) ? 0 : cs + 1;
#pragma unroll
    for (int ks = 0; ks + 1 < kKS; ++ks) {
      frags(w_rd + cs * kWTile + rd[ks + 1], a_rd + cs * kATile + rd[ks + 1], wb[(ks + 1) & 1], xa[(ks + 1) & 1]);
      lds_wait(true, wb[ks & 1], xa[ks & 1]);
      mfmas(wb[ks & 1], xa[ks & 1]);
    }
    lds_wait(false, wb[1], xa[1]);   // (kKS is even: the last k-step uses set 1, the next tile starts in set 0)
    if (t + 1 < nk) {
      // tiles t+1 .. t+NS-1 are outstanding; all but the first may stay in flight
      if (t + NS - 1 < nk) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads * (NS - 2)));
      else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
      wg_barrier();
      if (t + NS < nk) issue(t + NS, cs);
      frags(w_rd + ns * kWTile + rd[0], a_rd + ns * kATile + rd[0], wb[0], xa[0]);
    }
    __builtin_amdgcn_sched_barrier(0);
    mfmas(wb[1], xa[1]);
    cs = ns;
  }

  wg_barrier();   // every wave has read its last fragments (and no load is in flight): the ring is free
  if constexpr (SK) {
    if (!splitk_handover<1>(p, acc, (int64_t)tm * p.tiles_n + tn, z, wave, lane)) return;
  }
  store_wave_block<ACT, 1, BF>(p, acc, (lds_byte*)a_lds + wave * 4096, m0 + 32 * wt, n0 + 64 * wf, lane);
}

// ------------------------------------------------------------------------------------------
// C[M,N] = LN(A @ Wt^T + bias + residual) * gamma + beta, N = 256 * NC, one workgroup of 8
// waves per 64 token rows; wave w owns features [32*NC*w, 32*NC*(w+1)).  K tile = 32.
// ------------------------------------------------------------------------------------------
struct LnGemmParams {
  const half_t* A; const half_t* W; const half_t* bias; const half_t* res;
  const half_t* gamma; const half_t* beta; half_t* C;
  int M, N, K; float eps; float inv_n;
};

constexpr int kLM = 64;    // token rows per workgroup
constexpr int kLK = 32;    // K per tile: rows of 64 B, 4 chunks of 16 B

template <int NC>
__global__ __launch_bounds__(512) void gemm_bias_res_ln_kernel(const LnGemmParams p) {
  constexpr int N = 256 * NC;
  constexpr int kWTile = N * kLK * 2;      // weight tile bytes: 16 KB * NC
  constexpr int kATile = kLM * kLK * 2;    // 4 KB
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds0[kWTile];
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds1[kWTile];
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds0[kATile];
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds1[kATile];
  __shared__ float red[2][8][kLM];         // per-wave partial sums for mean / variance

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.x * kLM;

  // DMA: one instruction = 16 rows of 64 B.  Weight tile: 16*NC instructions, 2*NC per wave
  // (its OWN feature rows: wave w reads back exactly what it loaded, plus the shared A tile);
  // A tile: 4 instructions, issued by waves 0..3.
  const int drow = lane >> 2;                    // row within the instruction's 16
  uint32_t w_off[2 * NC];
#pragma unroll
  for (int i = 0; i < 2 * NC; ++i) {
    const int trow = 16 * (2 * NC * wave + i) + drow;     // feature index (< N)
    const int chunk = (lane & 3) ^ swz4(trow);
    w_off[i] = (uint32_t)trow * (uint32_t)(p.K * 2) + 16 * chunk;
  }
  uint32_t a_off;
  {
    const int trow = 16 * (wave & 3) + drow;
    const int chunk = (lane & 3) ^ swz4(trow);
    a_off = (uint32_t)min(trow, p.M - 1 - m0) * (uint32_t)(p.K * 2) + 16 * chunk;
  }
  const __amdgpu_buffer_rsrc_t a_rs = tile_rsrc(p.A + (int64_t)m0 * p.K), w_rs = tile_rsrc(p.W);
  auto issue = [&](int kt, lds_byte* wd, lds_byte* ad) {
    const uint32_t koff = (uint32_t)kt * (kLK * 2);
#pragma unroll
    for (int i = 0; i < 2 * NC; ++i) dma16b(w_rs, w_off[i], koff, wd + (2 * NC * wave + i) * 1024);
    if (wave < 4) dma16b(a_rs, a_off, koff, ad + wave * 1024);
  };
  // fragment read: row (32*t + j32), chunk 2*ks + g of 4, row pitch 64 B
  int rd[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) rd[ks] = j32 * 64 + (((2 * ks + g) ^ swz4(j32)) << 4);

  floatx16 acc[NC][2];   // [feature tile ni][token tile mi]
#pragma unroll
  for (int i = 0; i < NC; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  auto compute = [&](const lds_byte* wt, const lds_byte* at) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      half8_t xa[2];
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) xa[mi] = lds_frag(at, (32 * mi) * 64 + rd[ks]);
#pragma unroll
      for (int ni = 0; ni < NC; ++ni) {
        const half8_t wb = lds_frag(wt, (32 * NC * wave + 32 * ni) * 64 + rd[ks]);
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) acc[ni][mi] = mfma32<false>(wb, xa[mi], acc[ni][mi]);
      }
    }
  };

  const int nk = p.K / kLK;
  issue(0, (lds_byte*)w_lds0, (lds_byte*)a_lds0);
  for (int kt = 0; kt < nk; kt += 2) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (kt + 1 < nk) issue(kt + 1, (lds_byte*)w_lds1, (lds_byte*)a_lds1);
    compute((const lds_byte*)w_lds0, (const lds_byte*)a_lds0);
    if (kt + 1 < nk) {   // (no early exit from the loop: a second exit makes the compiler copy the accumulators)
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (kt + 2 < nk) issue(kt + 2, (lds_byte*)w_lds0, (lds_byte*)a_lds0);
      compute((const lds_byte*)w_lds1, (const lds_byte*)a_lds1);
    }
  }

  // ---- epilogue.  acc[ni][mi][r] = X[m0 + 32mi + j32][nb + 32ni + 8(r/4) + 4g + r%4],
  // nb = 32*NC*wave.  Add bias and residual, then LayerNorm over the full row.
  const int nb = 32 * NC * wave;
  float psum[2] = {0.f, 0.f};
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    const int m = min(m0 + 32 * mi + j32, p.M - 1);
#pragma unroll
    for (int ni = 0; ni < NC; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = nb + 32 * ni + 8 * q4 + 4 * g;
        half4_t bv = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        half4_t rv = bv;
        if (p.bias) bv = *reinterpret_cast<const half4_t*>(p.bias + n);
        if (p.res) rv = *reinterpret_cast<const half4_t*>(p.res + (int64_t)m * N + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = acc[ni][mi][4 * q4 + e] + (float)bv[e] + (float)rv[e];
          acc[ni][mi][4 * q4 + e] = x;
          psum[mi] += x;
        }
      }
    psum[mi] = pair_sum(psum[mi]);
  }
  if (g == 0) { red[0][wave][j32] = psum[0]; red[0][wave][32 + j32] = psum[1]; }
  __syncthreads();
  float mean[2], rstd[2];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) s += red[0][w][32 * mi + j32];
    mean[mi] = s * p.inv_n;
  }
  float pvar[2] = {0.f, 0.f};
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
    for (int ni = 0; ni < NC; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) { const float d = acc[ni][mi][r] - mean[mi]; pvar[mi] += d * d; }
    pvar[mi] = pair_sum(pvar[mi]);
  }
  if (g == 0) { red[1][wave][j32] = pvar[0]; red[1][wave][32 + j32] = pvar[1]; }
  __syncthreads();
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) s += red[1][w][32 * mi + j32];
    rstd[mi] = 1.0f / sqrtf(s * p.inv_n + p.eps);
  }
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    const int m = m0 + 32 * mi + j32;
    if (m >= p.M) continue;
    half_t* crow = p.C + (int64_t)m * N;
#pragma unroll
    for (int ni = 0; ni < NC; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = nb + 32 * ni + 8 * q4 + 4 * g;
        half4_t gv = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
        half4_t tv = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        if (p.gamma) gv = *reinterpret_cast<const half4_t*>(p.gamma + n);
        if (p.beta) tv = *reinterpret_cast<const half4_t*>(p.beta + n);
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (half_t)((acc[ni][mi][4 * q4 + e] - mean[mi]) * rstd[mi] * (float)gv[e] + (float)tv[e]);
        *reinterpret_cast<half4_t*>(crow + n) = o;
      }
  }
}

// ------------------------------------------------------------------------------------------
// The same operator on the 128 x 128 tiles of the bias / activation GEMM: the N / 128 workgroups
// that share a block of 128 token rows (a "row-block cluster") exchange per-row statistics
// through a small workspace instead of one workgroup owning the whole row.  The grid then fills
// the chip at 8192 tokens (hidden 768: 384 workgroups instead of 128) and every workgroup brings
// in one 128-wide slice of the weights, while the pre-normalisation values still never leave
// the registers.
//
//  * wave (wm, wn) of a workgroup holds 64 token rows x 64 features.  After bias and residual
//    (requested before the K loop, so their latency is hidden behind it) it forms mean and
//    M2 = sum (x - mean)^2 of its 64 values per row (two passes in registers) and publishes them
//    as ONE 8-byte word per row, stats[row block][part = 2 tn + wn][row], whose top bit (the sign
//    of M2, never set by the arithmetic) says "valid";
//  * it then reads the words of all 2 N / 128 parts of its rows until every one is valid - the
//    word itself is the signal, so nothing has to be ordered against anything else -, merges
//    them (equal counts: mean = average of the means, M2 = sum M2_i + 64 sum (mean_i - mean)^2),
//    normalises its registers and stores through LDS as full 128-byte lines;
//  * the words travel as relaxed device-scope atomic stores and loads: these are performed beyond
//    the XCD's cache, so no cache write-back or invalidate is needed (a device-scope fence would
//    write back the whole L2 of the XCD once per wave);
//  * the wait is bounded: after a fixed number of polls (2^18, or the caller's limit) the wave sets the error word of the
//    workspace and goes on (its output rows are then wrong, the launch still ends).  The cluster's
//    workgroups are 8 apart in dispatch order - round-robin over the 8 XCDs puts them on one XCD,
//    where they share the activation rows in L2.  The grid never exceeds two workgroups per
//    compute unit, which all run at once, and each walks over several tiles when there are more:
//    a workgroup then only waits for workgroups that are running.  (One workgroup per tile, with
//    more tiles than the chip holds, did run into the limit: once in some forty launches of
//    65536 x 1024 x 4096 a resident workgroup waited for one that had not been started.);
//  * having stored its output, a wave counts itself out of its half row block (64 rows); the
//    last one to leave puts the half's words and the counter back to zero, so the workspace
//    serves the next call as it is.
// ------------------------------------------------------------------------------------------
struct LnClusterParams {
  const half_t* A; const half_t* W; const half_t* bias; const half_t* res;
  const half_t* gamma; const half_t* beta; half_t* C;
  unsigned long long* stats;   // [tiles_m][2 * tiles_n][128] packed (mean, M2 | valid)
  int* departed;               // [tiles_m * 2]
  int* error;
  int M, N, K; int lda, ldr, ldc; float eps; float inv_n;
  int tiles_m, tiles_n; int spin_limit;
  int total_groups;            // tiles of the walk: tiles_m rounded up to 8, times tiles_n
};

constexpr int kClusterSpinLimit = 1 << 18;   // default number of polls before a wave gives up
constexpr unsigned long long kStatsValid = 1ull << 63;
// The waits of this kernel need every workgroup of the grid to be running: the grid is sized to
// kClusterGroupsPerCu workgroups per compute unit, which the launch bounds (registers) and the
// tile buffers (LDS) must allow; the host also asks the runtime what it allows (see the launch).
constexpr int kClusterGroupsPerCu = 2;
constexpr int kLdsPerCu = 160 * 1024;
static_assert(kClusterGroupsPerCu * 4 * kGTile <= kLdsPerCu, "the cluster kernel's tile buffers must fit a compute unit kClusterGroupsPerCu times");

template <int NT, bool BF = false>   // NT = N / 128 workgroups per row block
__global__ __launch_bounds__(256, kClusterGroupsPerCu) void gemm_bias_res_ln_cluster_kernel(const LnClusterParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds0[kGTile];
  __shared__ __attribute__((aligned(1024))) unsigned char a_lds1[kGTile];
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds0[kGTile];
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds1[kGTile];
  constexpr int kParts = NT;           // published words per row: one per workgroup of the row block (its 128 features)
  constexpr int kLeavers = 2 * NT;     // waves that read the words of a half row block (two feature halves per workgroup)

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31, g = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;

  int rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) rd[ks] = j32 * 128 + (((2 * ks + g) ^ swz(j32)) << 4);

  // The grid is never larger than what the chip holds at once (see the launch), and a workgroup
  // walks over tiles blockIdx, blockIdx + gridDim, ... (gridDim a multiple of 8, so a workgroup
  // stays with the token tiles of its XCD).  A workgroup only ever waits for workgroups that are
  // running, and no wait can close a circle: tile v waits for its partners v' < v + 8 NT, whose
  // workgroups first had to finish tile v' - gridDim < v (gridDim >= 8 NT), and so on downwards.
  for (int vb = blockIdx.x; vb < p.total_groups; vb += gridDim.x) {
  // tile index -> (XCD x, i): the NT workgroups of a row block are consecutive on one XCD
  const int x = vb & 7, i = vb >> 3;
  const int tn = i % NT;
  const int tm = (i / NT) * 8 + x;
  if (tm >= p.tiles_m) continue;   // (a whole cluster at a time: nobody waits for these)
  const int m0 = tm * kGT, n0 = tn * kGT;
  const int nb = n0 + 64 * wn;   // first feature of this wave

  // Bias of this lane's columns, in the accumulator layout
  // acc[ni][mi][r] = X[m0 + 64 wm + 32 mi + j32][nb + 32 ni + 8 (r / 4) + 4 g + r % 4]
  // (requested inside the K loop, so that neither the first tile's wait nor the epilogue sees
  // the latency).
  half4_t bv[2][4];
  auto request_bias = [&]() {
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        bv[ni][q4] = half4_t{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        if (p.bias) bv[ni][q4] = *reinterpret_cast<const half4_t*>(p.bias + nb + 32 * ni + 8 * q4 + 4 * g);
      }
  };
  // The residual tile (128 rows x 256 B) comes in like one more operand tile: as full lines,
  // direct to LDS, into the stage that the last K tile does not use, while that tile is being
  // multiplied.  (Read from global memory in the accumulator layout it would be 8 bytes out of
  // each of 32 rows per instruction, on the address path that already limits the K loop: measured
  // +3 us on the 8192 x 768 x 768 product.)  Rows 0-63 go to the stage's A buffer, rows 64-127 to
  // its W buffer; 16-byte chunk c of row r sits at chunk position c ^ (r & 15).
  auto issue_residual = [&](lds_byte* ad, lds_byte* wd) {
    if (!p.res) return;
    lds_byte* dst = (wave < 2 ? ad : wd) + (wave & 1) * 8192;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int row = 32 * wave + 4 * t + (lane >> 4);
      const int chunk = (lane & 15) ^ (row & 15);
      const int m = min(m0 + row, p.M - 1);
      dma16(p.res + (int64_t)m * p.ldr + n0 + 8 * chunk, dst + t * 1024);
    }
  };

  uint32_t a_off[4], w_off[4];
#pragma unroll
  for (int ii = 0; ii < 4; ++ii) {
    const int trow = 8 * (4 * wave + ii) + (lane >> 3);
    const int chunk = (lane & 7) ^ swz(trow);
    a_off[ii] = (uint32_t)min(trow, p.M - 1 - m0) * (uint32_t)(p.lda * 2) + 16 * chunk;   // rows past the edge re-read the last row
    w_off[ii] = (uint32_t)trow * (uint32_t)(p.K * 2) + 16 * chunk;
  }
  const __amdgpu_buffer_rsrc_t a_rs = tile_rsrc(p.A + (int64_t)m0 * p.lda), w_rs = tile_rsrc(p.W + (int64_t)n0 * p.K);
  auto issue = [&](int kt, lds_byte* ad, lds_byte* wd) {
    const uint32_t koff = (uint32_t)kt * (kGK * 2);
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) dma16b(a_rs, a_off[ii], koff, ad + (4 * wave + ii) * 1024);
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) dma16b(w_rs, w_off[ii], koff, wd + (4 * wave + ii) * 1024);
  };
  floatx16 acc[2][2];   // [feature tile ni][token tile mi]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // Fragments of k-step ks + 1 are requested before the MFMAs of k-step ks are issued (two sets of
  // fragment registers), so the LDS latency of a k-step hides behind the previous one's products.
  auto compute = [&](const lds_byte* at, const lds_byte* wt) {
    half8_t xa[2][2], wb[2][2];
    auto fetch = [&](int ks, int set) {
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) xa[set][mi] = lds_frag(at, (64 * wm + 32 * mi) * 128 + rd[ks]);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) wb[set][ni] = lds_frag(wt, (64 * wn + 32 * ni) * 128 + rd[ks]);
    };
    fetch(0, 0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) fetch(ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) acc[ni][mi] = mfma32<BF>(wb[ks & 1][ni], xa[ks & 1][mi], acc[ni][mi]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nk = p.K / kGK;
  const int res_at = nk > 2 ? 2 : 0;
  issue(0, (lds_byte*)a_lds0, (lds_byte*)w_lds0);
  for (int kt = 0; kt < nk; kt += 2) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (kt + 1 < nk) issue(kt + 1, (lds_byte*)a_lds1, (lds_byte*)w_lds1);
    else issue_residual((lds_byte*)a_lds1, (lds_byte*)w_lds1);   // tile kt is the last one
    if (kt == res_at) request_bias();
    compute((const lds_byte*)a_lds0, (const lds_byte*)w_lds0);
    if (kt + 1 < nk) {   // (no early exit from the loop: a second exit makes the compiler copy the accumulators)
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (kt + 2 < nk) issue(kt + 2, (lds_byte*)a_lds0, (lds_byte*)w_lds0);
      else issue_residual((lds_byte*)a_lds0, (lds_byte*)w_lds0);   // tile kt + 1 is the last one
      compute((const lds_byte*)a_lds1, (const lds_byte*)w_lds1);
    }
  }
  // The residual sits in the stage that did not hold the last tile; the other stage, free after
  // the barrier below, becomes the staging area of the output.
  const bool last_in_0 = (nk & 1) != 0;
  const lds_byte* res_lds = (const lds_byte*)(last_in_0 ? (wm ? w_lds1 : a_lds1) : (wm ? w_lds0 : a_lds0));
  lds_byte* stage = (lds_byte*)(last_in_0 ? a_lds0 : a_lds1) + wave * 4096;
  __builtin_amdgcn_s_waitcnt(0x0F70);   // this wave's share of the residual tile has landed
  __syncthreads();   // every wave is done with the operand tiles: they become the store staging

  // ---- bias + residual; statistics of this wave's 64 features per row
  float wmean[2], wm2[2];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    half4_t rv[2][4];
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int rowl = 32 * mi + j32, c = 8 * wn + 4 * ni + q4;
        rv[ni][q4] = half4_t{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        if (p.res) rv[ni][q4] = *reinterpret_cast<const __attribute__((address_space(3))) half4_t*>(res_lds + rowl * 256 + ((c ^ (rowl & 15)) << 4) + 8 * g);
      }
    float s = 0.f;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const half_t be = bv[ni][q4][e], re = rv[ni][q4][e];
          const float v = acc[ni][mi][4 * q4 + e] + from_elem<BF>(be) + from_elem<BF>(re);
          acc[ni][mi][4 * q4 + e] = v;
          s += v;
        }
    wmean[mi] = pair_sum(s) * (1.0f / 64.0f);
    float d2 = 0.f;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) { const float d = acc[ni][mi][r] - wmean[mi]; d2 += d * d; }
    wm2[mi] = pair_sum(d2);
  }

  // ---- the two waves of a row half (feature halves wn = 0, 1) first merge their statistics through
  // LDS (the W buffer of the last tile's stage is free since the barrier above): the workgroup then
  // publishes ONE word per row for its 128 features, a wave's own workgroup never costs it a trip
  // through memory, and a poll reads half as many words.  Lane (j32, g) speaks for row
  // 64 wm + 32 g + j32 of the row block.
  const int row_l = 64 * wm + 32 * g + j32;
  unsigned long long* my_stats = p.stats + ((int64_t)tm * (2 * NT)) * kGT + row_l;   // (the workspace keeps room for 2 NT words per row)
  float own_mean, own_m2;   // of this workgroup's 128 features
  {
    __attribute__((address_space(3))) float* xs = (__attribute__((address_space(3))) float*)(last_in_0 ? (lds_byte*)w_lds0 : (lds_byte*)w_lds1);
    const float pm = g ? wmean[1] : wmean[0], pq = g ? wm2[1] : wm2[0];
    xs[(2 * wn) * kGT + row_l] = pm;
    xs[(2 * wn + 1) * kGT + row_l] = pq;
    __syncthreads();
    const float om = xs[(2 * (1 - wn)) * kGT + row_l], oq = xs[(2 * (1 - wn) + 1) * kGT + row_l];
    const float ma = wn ? om : pm, mb = wn ? pm : om;   // (feature half 0, feature half 1: the same order in both waves)
    const float qa = wn ? oq : pq, qb = wn ? pq : oq;
    own_mean = 0.5f * (ma + mb);
    const float da = ma - own_mean, db = mb - own_mean;
    own_m2 = (qa + qb) + 64.0f * (da * da + db * db);
    if (wn == 0) {
      const unsigned long long word = ((unsigned long long)__builtin_bit_cast(unsigned, own_m2) << 32) | __builtin_bit_cast(unsigned, own_mean);
      __hip_atomic_store(my_stats + (int64_t)tn * kGT, word | kStatsValid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  // gamma and beta are requested here: they arrive while the wave waits for the other parts
  half4_t gv[2][4], tv[2][4];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int n = nb + 32 * ni + 8 * q4 + 4 * g;
      gv[ni][q4] = half4_t{to_elem<BF>(1.f), to_elem<BF>(1.f), to_elem<BF>(1.f), to_elem<BF>(1.f)};
      tv[ni][q4] = half4_t{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
      if (p.gamma) gv[ni][q4] = *reinterpret_cast<const half4_t*>(p.gamma + n);
      if (p.beta) tv[ni][q4] = *reinterpret_cast<const half4_t*>(p.beta + n);
    }

  // ---- collect the parts of this lane's row: read those of the other workgroups until all are valid
  unsigned long long word[kParts];
  {
    const unsigned long long own_word = (((unsigned long long)__builtin_bit_cast(unsigned, own_m2) << 32) | __builtin_bit_cast(unsigned, own_mean)) | kStatsValid;
    int polls = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int pt = 0; pt < kParts; ++pt) {
        word[pt] = own_word;
        if (pt != tn) word[pt] = __hip_atomic_load(my_stats + (int64_t)pt * kGT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = ok && (word[pt] & kStatsValid) != 0;
      }
      if (!__any(!ok)) break;
      if (++polls >= p.spin_limit) {
        if (lane == 0) __hip_atomic_store(p.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(4);
    }
  }
  float mean_own = 0.f, m2 = 0.f;
#pragma unroll
  for (int pt = 0; pt < kParts; ++pt) {
    mean_own += __builtin_bit_cast(float, (unsigned)(word[pt] & 0xffffffffull));
    m2 += __builtin_bit_cast(float, (unsigned)((word[pt] & ~kStatsValid) >> 32));
  }
  mean_own *= 1.0f / (float)kParts;
  float spread = 0.f;
#pragma unroll
  for (int pt = 0; pt < kParts; ++pt) {
    const float d = __builtin_bit_cast(float, (unsigned)(word[pt] & 0xffffffffull)) - mean_own;
    spread += d * d;
  }
  m2 += 128.0f * spread;   // (every part speaks for 128 features)
  const float rstd_own = 1.0f / sqrtf(m2 * p.inv_n + p.eps);
  const float mean_other = xchg32(mean_own), rstd_other = xchg32(rstd_own);
  float mean[2], rstd[2];
  mean[0] = g ? mean_other : mean_own; mean[1] = g ? mean_own : mean_other;
  rstd[0] = g ? rstd_other : rstd_own; rstd[1] = g ? rstd_own : rstd_other;

  // ---- normalise and store: each 32 x 64 block through 4 KB of LDS of the wave's own, out as
  // full 128-byte lines (see store_wave_block)
  const __amdgpu_buffer_rsrc_t c_rsrc = stof_wave_rsrc(p.C + (int64_t)(m0 + 64 * wm) * p.ldc + nb);
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const half_t ge = gv[ni][q4][e], te = tv[ni][q4][e];
          o[e] = to_elem<BF>((acc[ni][mi][4 * q4 + e] - mean[mi]) * rstd[mi] * from_elem<BF>(ge) + from_elem<BF>(te));
        }
        *reinterpret_cast<__attribute__((address_space(3))) half4_t*>(stage + j32 * 128 + (((4 * ni + q4) ^ (j32 & 7)) << 4) + 8 * g) = o;
      }
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      const int t = 8 * ii + (lane >> 3), c = lane & 7;
      const half8_t o = *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(stage + t * 128 + ((c ^ (t & 7)) << 4));
      const int m = m0 + 64 * wm + 32 * mi + t;
      if (m < p.M) stof_store16_through(c_rsrc, (uint32_t)(32 * mi + t) * (uint32_t)(p.ldc * 2) + 16 * c, o);
    }
  }

  // ---- leave; the last wave of the half row block zeroes its words and the counter.  (Every
  // wave that counts itself out has read all the parts, so nobody reads them after this.)
  int* dep = p.departed + (2 * tm + wm);
  int prev = 0;
  if (lane == 0) prev = __hip_atomic_fetch_add(dep, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  prev = __builtin_amdgcn_readfirstlane(prev);
  if (prev == kLeavers - 1) {
#pragma unroll
    for (int pt = 0; pt < kParts; ++pt)
      __hip_atomic_store(my_stats + (int64_t)pt * kGT, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (lane == 0) __hip_atomic_store(dep, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();   // the staging areas are operand buffers again
  }
}

// Workspace: error word (first 16 bytes), the counters of kClusterMaxRows / 128 row blocks, then
// the statistics.  The counter area has one size for every problem, so that a workspace that has
// served one shape can serve any other.  All of it is zero between calls.
constexpr int64_t kClusterMaxRows = 1 << 21;
constexpr int64_t kClusterStatsOffset = 16 + (kClusterMaxRows / kGT) * 8 + 240;   // a multiple of 256
static_assert(kClusterStatsOffset % 256 == 0, "statistics start on a 256-byte boundary");

// Which form runs.
//  * the 128 x 128 double-buffered form for almost everything.  With its tile loads through buffer
//    resources (no 64-bit vector add per load) and the banded tile order it is the fastest form
//    from 4096 rows up at every N and K measured (settled clocks, us, rows x N x K, against the
//    ring form with 256-token tiles and 3 stages): 8192 x 3072 x 768 45.6 vs 48.0, 8192 x 2304 x 768
//    36.2 vs 41.4, 8192 x 1024 x 4096 64.5 vs 73.3, 32768 x 3072 x 768 167 vs 185, 65536 x 3072 x 768
//    361 vs 372, 65536 x 768 x 3072 327 vs 359, 65536 x 1024 x 4096 549 vs 606 (1000 TFLOP/s),
//    8192^3 1042 vs 1095.  (Before these two changes the 256-token ring was the form for every
//    grid of 768+ workgroups, by 3-8 %; it is no longer chosen.);
//  * small ring (64-token tiles, 4 stages) when the 128 x 128 form would have at most
//    kSmallMaxTiles workgroups.  GPU time, N x K of the BERT-base layer: 512 tokens 14.4 -> 8.9,
//    14.0 -> 8.4, 14.5 -> 10.6, 36.0 -> 22.9 us; 2048 tokens x N 768: 14.2 -> 8.9, 36.9 -> 23.2 us;
//    from 192 tiles on (4096 tokens x N 768, 2048 x N 2304) the two are within 5 % either way.
constexpr int kSmallStages = 3;
constexpr int kSmallMaxTiles = 128;

// One launch of a bias / activation GEMM: tile form (64-token ring or 128 x 128), K split over
// workgroups or not, element format.
template <bool SMALL, bool SK, bool BF>
int launch_gemm(const GemmParams& p, int act, unsigned groups, hipStream_t st) {
  const dim3 grid(groups), block(256);
  switch (act) {
#define STOF_GEMM_CASE(A) \
    case A: \
      if constexpr (SMALL) hipLaunchKernelGGL((gemm_bias_act_ring_kernel<A, kSmallStages, SK, kSmallKT, BF>), grid, block, 0, st, p); \
      else hipLaunchKernelGGL((gemm_bias_act_kernel<A, SK, BF>), grid, block, 0, st, p); \
      break;
    STOF_GEMM_CASE(STOF_ACT_NONE)
    STOF_GEMM_CASE(STOF_ACT_GELU_ERF)
    STOF_GEMM_CASE(STOF_ACT_GELU_TANH)
    STOF_GEMM_CASE(STOF_ACT_RELU)
#undef STOF_GEMM_CASE
    default: return STOF_ERR_UNSUPPORTED;
  }
  return stof_check_launch();
}
template <bool SK>
int launch_gemm(const GemmParams& p, bool small, int dtype, int act, hipStream_t st) {
  const unsigned groups = raster_grid(p.tiles_m, p.tiles_n) * (unsigned)(SK ? p.splits : 1);
  if (dtype == STOF_DTYPE_BF16)
    return small ? launch_gemm<true, SK, true>(p, act, groups, st) : launch_gemm<false, SK, true>(p, act, groups, st);
  return small ? launch_gemm<true, SK, false>(p, act, groups, st) : launch_gemm<false, SK, false>(p, act, groups, st);
}

}  // namespace

extern "C" int stof_gemm_bias_act_dt(const void* A, const void* Wt, const void* bias, void* C,
                                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                                     int act, int dtype, void* stream) {
  if (!A || !Wt || !C) return STOF_ERR_NULL_POINTER;
  if (M <= 0 || N <= 0 || K <= 0 || K % kGK != 0 || N % 8 != 0 || lda < K || ldc < N) return STOF_ERR_BAD_SHAPE;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30) || ldc >= (1 << 23)) return STOF_ERR_BAD_SHAPE;   // (ldc: 32-bit byte offsets inside a wave's block of C)
  if (dtype != STOF_DTYPE_F16 && dtype != STOF_DTYPE_BF16) return STOF_ERR_UNSUPPORTED;
  if (!stof_aligned16(A) || !stof_aligned16(Wt) || !stof_aligned16(C) || (bias && ((uintptr_t)bias & 7)) ||
      lda % 8 != 0 || ldc % 8 != 0)
    return STOF_ERR_MISALIGNED;
  GemmParams p;
  p.A = (const half_t*)A; p.W = (const half_t*)Wt; p.bias = (const half_t*)bias; p.C = (half_t*)C;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = (int)lda; p.ldc = (int)ldc;
  p.partials = nullptr; p.counters = nullptr; p.splits = 1; p.nk_split = 0;
  if (((M + 63) / 64) * ((N + kGT - 1) / kGT) > (1 << 30)) return STOF_ERR_BAD_SHAPE;   // the grid is a 32-bit count
  const bool small = ((M + kGT - 1) / kGT) * ((N + kGT - 1) / kGT) <= kSmallMaxTiles;
  const int tile_m = small ? 64 : kGT;
  p.tiles_m = (int)((M + tile_m - 1) / tile_m); p.tiles_n = (int)((N + kGT - 1) / kGT);
  return launch_gemm<false>(p, small, dtype, act, (hipStream_t)stream);
}

extern "C" int stof_gemm_bias_act(const void* A, const void* Wt, const void* bias, void* C,
                                  int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                                  int act, void* stream) {
  return stof_gemm_bias_act_dt(A, Wt, bias, C, M, N, K, lda, ldc, act, STOF_DTYPE_F16, stream);
}

// ---- K split over workgroups (either tile form), for few output tiles and a long K --------------
// Workspace: one counter per (tile, wave) for up to kSplitMaxTiles tiles (a fixed area, so that a
// workspace that served one shape can serve another; zero between calls), then the fp32 partial
// sums: 32 KB per (64 x 128 tile, split) or 64 KB per (128 x 128 tile, split).
constexpr int64_t kSplitMaxTiles = 4096;
constexpr int64_t kSplitPartialsOffset = kSplitMaxTiles * 4 * 4;
constexpr int kSplitMaxSplits = 8;       // what the entry point takes
// What the plan chooses.  Measured on MI355X (us; one workgroup per tile, then 2 / 3 / 4 / 6 / 8 splits), GELU
// epilogue: 512 x 768 x 3072 22.2 | 15.7 13.7 13.9 19.6 17.0; 128 x 768 x 3072 21.3 | 14.8 13.0 12.7 18.1 15.9;
// 512 x 1024 x 4096 27.7 | 18.6 16.5 17.3 20.3 21.4; 1024 x 768 x 3072 21.8 | 15.9 22.8 17.7 22.0 20.9;
// 2048 x 768 x 3072 22.3 | 24.6 27.3 25.3; 512 x 768 x 768 7.7 | 8.6 8.7 8.9; 512 x 2304 x 768 8.3 | 12.4 12.0:
// (taken with 32-wide k-tiles) it pays while the grid stays within one workgroup per compute unit and a split keeps K >= 768;
// the hand-over (stores acknowledged, count, reads) costs about 5 us.
// Between kSmallMaxTiles and kSplitMidMaxTiles tiles of 128 x 128 (fewer workgroups than compute
// units) two splits of a long K pay on that form as well, by less, because a workgroup hands over
// 64 KB: 3072 x 768 x 3072 34.4 -> 28.0, 4096 x 768 x 3072 34.8 -> 29.6, 3072 x 1024 x 4096 40.2 -> 36.1;
// 5120 x 768 x 3072 (240 tiles) 35.7 -> 33.4, 4096 x 1024 x 4096 (256) 43.2 -> 42.6, K 1536: 17.0 -> 19.7.
constexpr int kSplitMidMaxTiles = 192;
constexpr int kSplitMidMinK = 3072;
constexpr int kSplitPlanMaxSplits = 3;   // (3 and 4 splits measure alike where 4 fit; 4 is the less steady)
constexpr int kSplitMinK = 768;          // K per split at least
constexpr int kSplitTargetGroups = 256;  // one workgroup per compute unit

// How many ways stof_gemm_bias_act_splitk should split K for this shape; 1 = the plain form is the
// one to use.  Mostly where the plain GEMM runs its 64-token form (at most kSmallMaxTiles tiles of
// 128 x 128): there a workgroup's K loop runs at the latency of its loads and most compute units
// have no workgroup at all.
extern "C" int stof_gemm_bias_act_splitk_plan(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % kGK != 0) return 1;
  const int64_t tiles128 = ((M + kGT - 1) / kGT) * ((N + kGT - 1) / kGT);
  if (tiles128 > kSmallMaxTiles) return (tiles128 <= kSplitMidMaxTiles && K >= kSplitMidMinK) ? 2 : 1;
  const int64_t tiles64 = ((M + 63) / 64) * ((N + kWFeat - 1) / kWFeat);
  int64_t splits = kSplitTargetGroups / tiles64;
  if (splits > K / kSplitMinK) splits = K / kSplitMinK;
  if (splits > kSplitPlanMaxSplits) splits = kSplitPlanMaxSplits;
  return splits < 2 ? 1 : (int)splits;
}

extern "C" int64_t stof_gemm_bias_act_splitk_workspace_bytes(int64_t M, int64_t N, int splits) {
  if (M <= 0 || N <= 0 || splits < 1 || splits > kSplitMaxSplits) return 0;
  const int64_t tiles64 = ((M + 63) / 64) * ((N + kWFeat - 1) / kWFeat);
  if (tiles64 > kSplitMaxTiles) return 0;
  // (either form: fp32 partial sums of the output padded to whole 128 x 128 tiles, per split)
  return kSplitPartialsOffset + ((M + kGT - 1) / kGT) * ((N + kGT - 1) / kGT) * splits * (kGT * kGT * 4);
}

extern "C" int stof_gemm_bias_act_splitk_dt(const void* A, const void* Wt, const void* bias, void* C,
                                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                                            int act, int splits, void* workspace, int64_t workspace_bytes,
                                            int dtype, void* stream) {
  if (!A || !Wt || !C || !workspace) return STOF_ERR_NULL_POINTER;
  if (M <= 0 || N <= 0 || K <= 0 || K % kGK != 0 || N % 8 != 0 || lda < K || ldc < N) return STOF_ERR_BAD_SHAPE;
  if (K > (1 << 30) || ldc >= (1 << 23) || splits < 2 || splits > kSplitMaxSplits) return STOF_ERR_BAD_SHAPE;
  if (dtype != STOF_DTYPE_F16 && dtype != STOF_DTYPE_BF16) return STOF_ERR_UNSUPPORTED;
  const int64_t tiles64 = ((M + 63) / 64) * ((N + kWFeat - 1) / kWFeat);
  if (tiles64 > kSplitMaxTiles) return STOF_ERR_UNSUPPORTED;
  if (!stof_aligned16(A) || !stof_aligned16(Wt) || !stof_aligned16(C) || (bias && ((uintptr_t)bias & 7)) ||
      ((uintptr_t)workspace & 15) || lda % 8 != 0 || ldc % 8 != 0)
    return STOF_ERR_MISALIGNED;
  if (workspace_bytes < stof_gemm_bias_act_splitk_workspace_bytes(M, N, splits)) return STOF_ERR_BAD_SHAPE;
  GemmParams p;
  p.A = (const half_t*)A; p.W = (const half_t*)Wt; p.bias = (const half_t*)bias; p.C = (half_t*)C;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = (int)lda; p.ldc = (int)ldc;
  p.counters = reinterpret_cast<int*>(workspace);
  p.partials = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kSplitPartialsOffset);
  // The tile form follows the plain GEMM's rule: 64-token tiles where the 128 x 128 form would
  // have at most kSmallMaxTiles workgroups.
  const bool small = ((M + kGT - 1) / kGT) * ((N + kGT - 1) / kGT) <= kSmallMaxTiles;
  const int tile_m = small ? 64 : kGT, tile_k = small ? kSmallKT : kGK;
  p.tiles_m = (int)((M + tile_m - 1) / tile_m); p.tiles_n = (int)((N + kGT - 1) / kGT);
  const int nk = (int)(K / tile_k);
  p.nk_split = (nk + splits - 1) / splits;
  p.splits = (nk + p.nk_split - 1) / p.nk_split;   // (every split has at least one k-tile)
  return launch_gemm<true>(p, small, dtype, act, (hipStream_t)stream);
}

extern "C" int stof_gemm_bias_act_splitk(const void* A, const void* Wt, const void* bias, void* C,
                                         int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                                         int act, int splits, void* workspace, int64_t workspace_bytes, void* stream) {
  return stof_gemm_bias_act_splitk_dt(A, Wt, bias, C, M, N, K, lda, ldc, act, splits, workspace, workspace_bytes, STOF_DTYPE_F16, stream);
}

extern "C" int stof_gemm_bias_res_ln(const void* A, const void* Wt, const void* bias, const void* residual,
                                     const void* gamma, const void* beta, void* C,
                                     int64_t M, int64_t N, int64_t K, float eps, void* stream) {
  if (!A || !Wt || !C) return STOF_ERR_NULL_POINTER;
  if (M <= 0 || K <= 0 || K % kLK != 0 || M > (1 << 30) || K > (1 << 30)) return STOF_ERR_BAD_SHAPE;
  if (N != 256 && N != 512 && N != 768 && N != 1024) return STOF_ERR_UNSUPPORTED;
  if (!stof_aligned16(A) || !stof_aligned16(Wt) || ((uintptr_t)C & 7) || ((uintptr_t)bias & 7) ||
      ((uintptr_t)residual & 7) || ((uintptr_t)gamma & 7) || ((uintptr_t)beta & 7) || K % 8 != 0)
    return STOF_ERR_MISALIGNED;
  LnGemmParams p;
  p.A = (const half_t*)A; p.W = (const half_t*)Wt; p.bias = (const half_t*)bias; p.res = (const half_t*)residual;
  p.gamma = (const half_t*)gamma; p.beta = (const half_t*)beta; p.C = (half_t*)C;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.eps = eps; p.inv_n = 1.0f / (float)N;
  const dim3 grid((unsigned)((M + kLM - 1) / kLM)), block(512);
  hipStream_t st = (hipStream_t)stream;
  switch (N) {
    case 256: hipLaunchKernelGGL(gemm_bias_res_ln_kernel<1>, grid, block, 0, st, p); break;
    case 512: hipLaunchKernelGGL(gemm_bias_res_ln_kernel<2>, grid, block, 0, st, p); break;
    case 768: hipLaunchKernelGGL(gemm_bias_res_ln_kernel<3>, grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL(gemm_bias_res_ln_kernel<4>, grid, block, 0, st, p); break;
  }
  return stof_check_launch();
}

namespace {
// Workgroups of one instantiation of the cluster kernel that run at once on the current device:
// what the runtime reports per compute unit (registers, LDS), capped at the kClusterGroupsPerCu the
// kernel was written for, times the compute units.  Asked once per device and instantiation.
constexpr int kMaxDevices = 64;
template <int NT, bool BF>
int64_t cluster_resident_groups() {
  static int cached[kMaxDevices] = {};   // 0 = not asked yet, -1 = the query failed
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int groups = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);   // (two threads that both find 0 store the same number)
  if (groups == 0) {
    int cus = 0, per_cu = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0 ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_bias_res_ln_cluster_kernel<NT, BF>, 256, 0) != hipSuccess || per_cu <= 0)
      groups = -1;
    else
      groups = (per_cu < kClusterGroupsPerCu ? per_cu : kClusterGroupsPerCu) * cus;
    __atomic_store_n(&cached[dev], groups, __ATOMIC_RELAXED);
  }
  return groups < 0 ? 0 : groups / 8 * 8;
}
}  // namespace

extern "C" int64_t stof_gemm_bias_res_ln_cluster_workspace_bytes(int64_t M, int64_t N) {
  if (M <= 0 || M > kClusterMaxRows || N <= 0 || N % kGT != 0) return 0;
  return kClusterStatsOffset + ((M + kGT - 1) / kGT) * (2 * (N / kGT)) * kGT * 8;
}

extern "C" int stof_gemm_bias_res_ln_cluster_dt(const void* A, const void* Wt, const void* bias, const void* residual,
                                                const void* gamma, const void* beta, void* C,
                                                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldr, int64_t ldc,
                                                float eps, void* workspace, int64_t workspace_bytes, int dtype, void* stream) {
  return stof_gemm_bias_res_ln_cluster_bounded(A, Wt, bias, residual, gamma, beta, C, M, N, K, lda, ldr, ldc, eps,
                                               workspace, workspace_bytes, dtype, 0, stream);
}

extern "C" int stof_gemm_bias_res_ln_cluster_bounded(const void* A, const void* Wt, const void* bias, const void* residual,
                                                     const void* gamma, const void* beta, void* C,
                                                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldr, int64_t ldc,
                                                     float eps, void* workspace, int64_t workspace_bytes, int dtype,
                                                     int spin_limit, void* stream) {
  if (!A || !Wt || !C || !workspace) return STOF_ERR_NULL_POINTER;
  if (spin_limit < 0) return STOF_ERR_BAD_SHAPE;
  if (dtype != STOF_DTYPE_F16 && dtype != STOF_DTYPE_BF16) return STOF_ERR_UNSUPPORTED;
  if (M <= 0 || K <= 0 || K % kGK != 0 || M > kClusterMaxRows || K > (1 << 30) || lda < K || ldc < N || ldc >= (1 << 23) || (residual && ldr < N))
    return STOF_ERR_BAD_SHAPE;
  if (N % kGT != 0 || N < 2 * kGT || N > 8 * kGT) return STOF_ERR_UNSUPPORTED;   // 256, 384, ..., 1024
  if (!stof_aligned16(A) || !stof_aligned16(Wt) || !stof_aligned16(C) || ((uintptr_t)bias & 7) ||
      !stof_aligned16(residual) || ((uintptr_t)gamma & 7) || ((uintptr_t)beta & 7) || ((uintptr_t)workspace & 15) ||
      lda % 8 != 0 || ldc % 8 != 0 || ldr % 8 != 0)
    return STOF_ERR_MISALIGNED;
  if (workspace_bytes < stof_gemm_bias_res_ln_cluster_workspace_bytes(M, N)) return STOF_ERR_BAD_SHAPE;
  LnClusterParams p;
  p.A = (const half_t*)A; p.W = (const half_t*)Wt; p.bias = (const half_t*)bias; p.res = (const half_t*)residual;
  p.gamma = (const half_t*)gamma; p.beta = (const half_t*)beta; p.C = (half_t*)C;
  p.tiles_m = (int)((M + kGT - 1) / kGT); p.tiles_n = (int)(N / kGT);
  p.error = reinterpret_cast<int*>(workspace);
  p.departed = p.error + 4;
  p.stats = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(workspace) + kClusterStatsOffset);
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = (int)lda; p.ldr = (int)ldr; p.ldc = (int)ldc;
  p.eps = eps; p.inv_n = 1.0f / (float)N; p.spin_limit = spin_limit == 0 ? kClusterSpinLimit : spin_limit;
  const int64_t groups = (int64_t)((p.tiles_m + 7) / 8) * 8 * p.tiles_n;
  if (groups > (1 << 30)) return STOF_ERR_BAD_SHAPE;
  p.total_groups = (int)groups;
  // A grid of at most the workgroups that run at once (a multiple of 8) is running as a whole
  // from the start; fewer than one cluster per XCD, or a runtime that will not say: not this form.
  hipStream_t st = (hipStream_t)stream;
  const bool bf = dtype == STOF_DTYPE_BF16;
  switch (p.tiles_n) {
#define STOF_CLUSTER_CASE(NT) \
    case NT: { \
      const int64_t resident = bf ? cluster_resident_groups<NT, true>() : cluster_resident_groups<NT, false>(); \
      if (resident < 8 * p.tiles_n) return STOF_ERR_UNSUPPORTED; \
      const dim3 grid((unsigned)(groups < resident ? groups : resident)), block(256); \
      if (bf) hipLaunchKernelGGL((gemm_bias_res_ln_cluster_kernel<NT, true>), grid, block, 0, st, p); \
      else hipLaunchKernelGGL((gemm_bias_res_ln_cluster_kernel<NT, false>), grid, block, 0, st, p); \
      break; }
    STOF_CLUSTER_CASE(2) STOF_CLUSTER_CASE(3) STOF_CLUSTER_CASE(4) STOF_CLUSTER_CASE(5)
    STOF_CLUSTER_CASE(6) STOF_CLUSTER_CASE(7) STOF_CLUSTER_CASE(8)
#undef STOF_CLUSTER_CASE
    default: return STOF_ERR_UNSUPPORTED;
  }
  return stof_check_launch();
}

extern "C" int stof_gemm_bias_res_ln_cluster(const void* A, const void* Wt, const void* bias, const void* residual,
                                             const void* gamma, const void* beta, void* C,
                                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldr, int64_t ldc,
                                             float eps, void* workspace, int64_t workspace_bytes, void* stream) {
  return stof_gemm_bias_res_ln_cluster_dt(A, Wt, bias, residual, gamma, beta, C, M, N, K, lda, ldr, ldc, eps,
                                          workspace, workspace_bytes, STOF_DTYPE_F16, stream);
}
