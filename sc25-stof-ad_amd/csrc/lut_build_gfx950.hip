// Dense 0/1 mask -> block LUT on the GPU, for gfx950.
//
// Replaces the host loop of get_sparse_storage (src/util/masks.py:145-170: one torch.all per
// (query block, key block) pair, list appends, host -> device copies) with two launches:
//
//  1. classify: one wavefront per block_m x block_n tile reads the tile once with 16-byte loads
//     and decides with two wave-wide votes whether every element is 1 (FULL), every element is 0
//     (absent) or neither (PARTIAL); for 64 x 64 tiles it forms, in the same pass, the tile's 64
//     bit rows (bit j of row i = key j allowed) from the lanes' 16-byte chunks by lane exchanges.
//     One byte per tile (and 512 B of bit rows per partial tile) go to a scratch buffer.  This
//     pass moves the whole mask once and is bound by HBM bandwidth.
//  2. compact: one workgroup per row of tiles counts the FULL / PARTIAL tiles of the rows above
//     it (the class bytes: a few KB, L2-resident), ranks its own tiles with wave votes, and
//     writes its slice of the three CSR lists (row pointers, ascending key-block indices) and
//     the bit rows of its partial tiles into their PART slots.
//
// A third kernel writes, on request, the reference's additive fp16 blocks
// -10000 * (1 - block.half()) (src/util/masks.py:159-166) for the PART list.
//
// The scratch buffer is either passed in by the caller (stof_build_lut) or a fixed array in
// device memory (stof_build_lut_static), for callers that cannot allocate.
#include "stof_common.h"

// Scratch of stof_build_lut_static, the entry point that allocates nothing: class bytes and bit
// rows for at most kStaticMaxTiles tiles (8.05 MiB per GPU with the per-tile counts, held until the process ends).  In
// host code the array's name is a stand-in, not a device address: the address of each device's
// copy is taken once per device with hipGetSymbolAddress and only that pointer is used.
constexpr int64_t kStaticMaxTiles = 16384;   // S = 8192 at 64 x 64 blocks
constexpr int64_t kClsBytesStatic = kStaticMaxTiles;
constexpr int64_t kBitsBytesStatic = kStaticMaxTiles * 64 * 8;
constexpr int64_t kCntBytesStatic = kStaticMaxTiles * 2 + 16;   // non-zero count per tile, then the total (see LutParams)
static __device__ __align__(256) unsigned char scratch[kClsBytesStatic + kBitsBytesStatic + kCntBytesStatic];

namespace {

enum { kClsEmpty = 0, kClsFull = 1, kClsPart = 2 };

struct LutParams {
  const void* mask; int64_t ld;           // row pitch in elements
  int S, bm, bn, nQ, nK;
  unsigned char* cls; uint64_t* ws_bits;  // scratch: class byte per tile; 64 bit rows per tile (64 x 64 only, else null)
  unsigned short* cnt; long long* nnz;    // scratch: non-zero elements per tile (or null); their sum, written by the first row's workgroup
  int32_t* frp; int32_t* fci; int32_t* prp; int32_t* pci; int32_t* lrp; int32_t* lci;
  uint64_t* pbits;                        // [cap_part][64] or null
  int32_t* counts;                        // {n_full, n_part, n_load, overflow} or null
  int64_t cap_full, cap_part, cap_load;
};

__device__ __forceinline__ half_t additive_of(half_t x) {
  // -10000 * (1 - x) in fp16 arithmetic, as the reference forms it (src/util/masks.py:160)
  return (half_t)-10000.0f * ((half_t)1.0f - x);
}

// Eight consecutive elements of a tile row (one 16-byte load of fp16, two of fp32, both requested
// before the first compare): updates the two "every element is ..." votes and returns the keep
// bits (bit e = element e allowed, by the rule the bit rows are packed with elsewhere: additive
// value above -5000).
// Flag words of a lane over the elements it has looked at, kept as integers (a test per element on
// the bit patterns costs half the instructions of float compares and per-lane booleans):
//   nz   OR of the patterns without their sign bits  -> non-zero iff some element is not +-0
//   ne1  OR of (pattern XOR pattern of 1.0)          -> non-zero iff some element is not 1.0
//   cnt  non-zero elements (fp16: two 16-bit counters side by side, at most 64 x 2 per lane and call site)
struct ChunkFlags { uint32_t nz, ne1, cnt; };

template <typename T>
__device__ __forceinline__ uint32_t chunk_bits(const T* src, ChunkFlags& fl) {
  constexpr int E = 16 / (int)sizeof(T);      // elements per 16-byte load
  constexpr int L = 8 / E;                    // loads per eight elements
  typedef T vec_t __attribute__((ext_vector_type(E)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  vec_t x[L];
#pragma unroll
  for (int l = 0; l < L; ++l) x[l] = *reinterpret_cast<const vec_t*>(src + l * E);
  uint32_t cb = 0;
#pragma unroll
  for (int l = 0; l < L; ++l) {
    const u32x4 d = __builtin_bit_cast(u32x4, x[l]);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if constexpr (sizeof(T) == 2) {
        const uint32_t a = d[w] & 0x7FFF7FFFu;            // two halves without their signs
        fl.nz |= a;
        fl.ne1 |= d[w] ^ 0x3C003C00u;
        const u16x2 one = {1, 1};
        const u16x2 a2 = __builtin_bit_cast(u16x2, a);
        const u16x2 m = __builtin_elementwise_min(a2, one);   // 1 per non-zero half
        fl.cnt = __builtin_bit_cast(uint32_t, (u16x2)(__builtin_bit_cast(u16x2, fl.cnt) + m));
      } else {
        const uint32_t a = d[w] << 1;                     // the pattern without its sign
        fl.nz |= a;
        fl.ne1 |= d[w] ^ 0x3F800000u;
        fl.cnt += a != 0u;
      }
    }
#pragma unroll
    for (int e = 0; e < E; ++e)
      // (allowed = the additive value -10000 * (1 - x), formed in fp16, is above -5000: for every fp16 x
      // that is the same as x > 0.5, checked over all 65536 patterns; NaN is not allowed either way)
      cb |= (uint32_t)((half_t)x[l][e] > (half_t)0.5f) << (l * E + e);
  }
  return cb;
}

// T = half_t or float.  One wavefront per tile; a lane takes eight elements (one byte of a bit row) at a time.
template <typename T>
__global__ __launch_bounds__(256) void lut_classify_kernel(const LutParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= (int64_t)p.nQ * p.nK) return;
  const int r = (int)(tile / p.nK), c = (int)(tile - (int64_t)r * p.nK);
  const T* base = reinterpret_cast<const T*>(p.mask) + (int64_t)r * p.bm * p.ld + (int64_t)c * p.bn;
  ChunkFlags fl = {0u, 0u, 0u};   // this lane's share of the tile (merged over the wave at the end)
  if (p.ws_bits) {
    // 64 x 64 tile: 8 lanes hold one row of 64 keys, a pass covers 8 rows, 8 passes.  (fp32 read
    // four elements per lane at first: twice the passes and lane exchanges for the same bytes,
    // and a larger mask ran slower per byte than the fp16 one.)
    constexpr int CPR = 8, PASSES = 8, ROWS = 8;
    const int ch = lane & (CPR - 1), row_in_pass = lane / CPR;
    uint64_t words[PASSES];   // lanes with chunk 0: the bit row of (pass, row_in_pass)
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const uint32_t cb = chunk_bits<T>(base + (int64_t)(ps * ROWS + row_in_pass) * p.ld + ch * 8, fl);
      const int sh = ch * 8;
      uint32_t lo = sh < 32 ? cb << sh : 0u, hi = sh >= 32 ? cb << (sh - 32) : 0u;
#pragma unroll
      for (int m = 1; m < CPR; m <<= 1) {
        lo |= (uint32_t)__shfl_xor((int)lo, m, 64);
        hi |= (uint32_t)__shfl_xor((int)hi, m, 64);
      }
      words[ps] = ((uint64_t)hi << 32) | lo;
    }
    const bool full = __ballot(fl.ne1 != 0u) == 0ull, empty = __ballot(fl.nz != 0u) == 0ull;
    if (lane == 0) p.cls[tile] = (unsigned char)(empty ? kClsEmpty : (full ? kClsFull : kClsPart));
    if (!full && !empty && ch == 0) {
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) p.ws_bits[tile * 64 + ps * ROWS + row_in_pass] = words[ps];
    }
  } else {
    const int cpr = p.bn / 8;                 // eight-element chunks per tile row
    const int total = p.bm * cpr;
    for (int idx = lane; idx < total; idx += 64) {
      const int row = idx / cpr, ch = idx - row * cpr;
      chunk_bits<T>(base + (int64_t)row * p.ld + ch * 8, fl);
    }
    const bool full = __ballot(fl.ne1 != 0u) == 0ull, empty = __ballot(fl.nz != 0u) == 0ull;
    if (lane == 0) p.cls[tile] = (unsigned char)(empty ? kClsEmpty : (full ? kClsFull : kClsPart));
  }
  if (p.cnt) {   // (at most 128 x 128 = 16384 per tile)
    int nonzero = sizeof(T) == 2 ? (int)((fl.cnt & 0xFFFFu) + (fl.cnt >> 16)) : (int)fl.cnt;
    for (int o = 32; o > 0; o >>= 1) nonzero += __shfl_xor(nonzero, o, 64);
    if (lane == 0) p.cnt[tile] = (unsigned short)nonzero;
  }
}

__device__ __forceinline__ int block_sum(int v, int* lds) {
  // sum over the 256 threads of the workgroup; lds: 4 ints
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  return lds[0] + lds[1] + lds[2] + lds[3];
}

__global__ __launch_bounds__(256) void lut_compact_kernel(const LutParams p) {
  __shared__ int red[4];
  __shared__ int wave_cnt[2][4];
  __shared__ int part_col[256], part_slot[256];   // this chunk's partial tiles, in column order
  const int r = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // FULL and PARTIAL tiles of the rows above: the class bytes (0, 1, 2) four at a time
  int nf = 0, np = 0;
  const int64_t above = (int64_t)r * p.nK;
  const uint32_t* cls4 = reinterpret_cast<const uint32_t*>(p.cls);   // (the class array is 4-byte aligned)
  for (int64_t i = tid; i < (above >> 2); i += 256) {
    const uint32_t x = cls4[i];
    nf += __builtin_popcount(x & 0x01010101u); np += __builtin_popcount(x & 0x02020202u);
  }
  if (tid < (int)(above & 3)) {
    const int c = p.cls[(above & ~(int64_t)3) + tid];
    nf += c == kClsFull; np += c == kClsPart;
  }
  int fbase = block_sum(nf, red);
  int pbase = block_sum(np, red);
  const unsigned char* row_cls = p.cls + above;
  for (int c0 = 0; c0 < p.nK; c0 += 256) {
    const int c = c0 + tid;
    const int cl = c < p.nK ? row_cls[c] : kClsEmpty;
    const uint64_t bf = __ballot(cl == kClsFull), bp = __ballot(cl == kClsPart);
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    if (lane == 0) { wave_cnt[0][wave] = __builtin_popcountll(bf); wave_cnt[1][wave] = __builtin_popcountll(bp); }
    __syncthreads();
    int f_before = 0, p_before = 0, f_all = 0, p_all = 0;
    for (int w = 0; w < 4; ++w) {
      if (w < wave) { f_before += wave_cnt[0][w]; p_before += wave_cnt[1][w]; }
      f_all += wave_cnt[0][w]; p_all += wave_cnt[1][w];
    }
    const int pl = p_before + __builtin_popcountll(bp & below);   // rank among this chunk's partial tiles
    const int rf = fbase + f_before + __builtin_popcountll(bf & below);
    const int rp = pbase + pl;
    if (cl == kClsFull) {
      if (rf < p.cap_full) p.fci[rf] = c;
      if (rf + rp < p.cap_load) p.lci[rf + rp] = c;
    } else if (cl == kClsPart) {
      part_col[pl] = c;
      part_slot[pl] = rp < p.cap_part ? rp : -1;
      if (rp < p.cap_part) p.pci[rp] = c;
      if (rf + rp < p.cap_load) p.lci[rf + rp] = c;
    }
    __syncthreads();
    // bit rows of this chunk's partial tiles into their PART slots (a wavefront per tile)
    if (p.pbits && p.ws_bits) {
      for (int t = wave; t < p_all; t += 4) {
        const int slot = part_slot[t];
        if (slot >= 0) p.pbits[(int64_t)slot * 64 + lane] = p.ws_bits[(above + part_col[t]) * 64 + lane];
      }
    }
    fbase += f_all; pbase += p_all;
    __syncthreads();
  }
  if (r == 0 && p.cnt && p.nnz) {
    // the mask's non-zero elements: the per-tile counts of the classify pass, summed by this one workgroup
    // (that of the first row of tiles, which has no rows above it to count: the last row's has the most)
    long long total = 0;
    const int64_t tiles = (int64_t)p.nQ * p.nK;
    // eight counts per 16-byte load (the count array starts 16-byte aligned), all of a thread's loads independent
    typedef unsigned short ushort8v __attribute__((ext_vector_type(8)));
    const int64_t vecs = tiles >> 3;
    for (int64_t i = tid; i < vecs; i += 256) {
      const ushort8v c8 = *reinterpret_cast<const ushort8v*>(p.cnt + 8 * i);
#pragma unroll
      for (int e = 0; e < 8; ++e) total += c8[e];
    }
    for (int64_t i = 8 * vecs + tid; i < tiles; i += 256) total += p.cnt[i];
    for (int o = 32; o > 0; o >>= 1) total += __shfl_xor(total, o, 64);
    __shared__ long long part_sum[4];
    __syncthreads();
    if (lane == 0) part_sum[wave] = total;
    __syncthreads();
    if (tid == 0) {
      const long long all = part_sum[0] + part_sum[1] + part_sum[2] + part_sum[3];
      *p.nnz = all;
      // the reference's figure (src/util/masks.py:137) in its own arithmetic: count / (S * S) * 100 in fp32
      reinterpret_cast<float*>(p.nnz + 1)[0] = (float)all / (float)((long long)p.S * p.S) * 100.0f;
    }
  }
  if (tid == 0) {
    if (r == 0) { p.frp[0] = 0; p.prp[0] = 0; p.lrp[0] = 0; }
    p.frp[r + 1] = fbase; p.prp[r + 1] = pbase; p.lrp[r + 1] = fbase + pbase;
    if (r == p.nQ - 1 && p.counts) {
      p.counts[0] = fbase; p.counts[1] = pbase; p.counts[2] = fbase + pbase;
      p.counts[3] = (fbase > p.cap_full || pbase > p.cap_part || fbase + pbase > p.cap_load) ? 1 : 0;
    }
  }
}

// out[s] = -10000 * (1 - block.half()) for PART slot s: (row from the PART row pointers, column pci[s]).
template <typename T>
__global__ __launch_bounds__(256) void lut_additive_blocks_kernel(const void* mask, int64_t ld, int bm, int bn, int nQ,
                                                                  const int32_t* __restrict__ prp, const int32_t* __restrict__ pci,
                                                                  half_t* __restrict__ out) {
  __shared__ int s_row;
  const int s = blockIdx.x;
  if (threadIdx.x == 0) {
    int lo = 0, hi = nQ;           // last r with prp[r] <= s
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (prp[mid] <= s) lo = mid; else hi = mid; }
    s_row = lo;
  }
  __syncthreads();
  const int r = s_row, c = pci[s];
  const T* base = reinterpret_cast<const T*>(mask) + (int64_t)r * bm * ld + (int64_t)c * bn;
  half_t* o = out + (int64_t)s * bm * bn;
  for (int i = threadIdx.x; i < bm * bn; i += 256) {
    const int row = i / bn, col = i - row * bn;
    o[i] = additive_of((half_t)base[(int64_t)row * ld + col]);
  }
}

// A LUT built with another block size (the reference's launcher takes BLOCK_M in {16, 32, 64} and
// BLOCK_N in {16 .. 128}, block_attn_mask_cuda.cu:6064-6322) described again with 64 x 64 tiles,
// the one shape the attention kernel has: full source block -> ones, partial source block -> the
// bits of its additive fp16 values, absent -> zeros.  One wavefront per 64 x 64 target tile, lane l
// forms the 64-bit row 64 I + l from the (at most four) source blocks it crosses, looked up by
// binary search in the source row's FULL and PART lists; the tile's class byte and bit rows go to
// the same scratch lut_compact_kernel reads, so the lists come out exactly as if the dense mask
// had been classified at 64 x 64.
struct RetileParams {
  const int32_t* frp; const int32_t* fci; const int32_t* prp; const int32_t* pci; const half_t* pbm;
  int bm, bn, n64;                       // source block shape; 64 x 64 tiles per side
  unsigned char* cls; uint64_t* ws_bits;
};

__device__ __forceinline__ int find_col(const int32_t* __restrict__ ci, int lo, int hi, int col) {
  // position of `col` in the ascending list ci[lo, hi), or -1
  while (lo < hi) { const int mid = (lo + hi) >> 1; const int v = ci[mid]; if (v == col) return mid; if (v < col) lo = mid + 1; else hi = mid; }
  return -1;
}

__global__ __launch_bounds__(256) void lut_retile_kernel(const RetileParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= (int64_t)p.n64 * p.n64) return;
  const int I = (int)(tile / p.n64), J = (int)(tile - (int64_t)I * p.n64);
  const int row = 64 * I + lane;
  const int ib = row / p.bm, ri = row - ib * p.bm;
  const int f0 = p.frp[ib], f1 = p.frp[ib + 1], q0 = p.prp[ib], q1 = p.prp[ib + 1];
  uint64_t word = 0;
  for (int jb = (64 * J) / p.bn; jb * p.bn < 64 * J + 64; ++jb) {
    const int c_lo = max(64 * J, jb * p.bn), c_hi = min(64 * J + 64, (jb + 1) * p.bn);
    const int w = c_hi - c_lo;
    uint64_t bits = 0;
    if (find_col(p.fci, f0, f1, jb) >= 0) {
      bits = w == 64 ? ~0ull : ((1ull << w) - 1);
    } else {
      const int slot = find_col(p.pci, q0, q1, jb);
      if (slot >= 0) {
        const half_t* src = p.pbm + ((int64_t)slot * p.bm + ri) * p.bn + (c_lo - jb * p.bn);   // (a multiple of 16 elements)
        for (int e0 = 0; e0 < w; e0 += 8) {
          const half8_t x = *reinterpret_cast<const half8_t*>(src + e0);
#pragma unroll
          for (int e = 0; e < 8; ++e) bits |= (uint64_t)((float)x[e] > -5000.0f) << (e0 + e);
        }
      }
    }
    word |= bits << (c_lo - 64 * J);
  }
  const bool full = __ballot(word != ~0ull) == 0ull, empty = __ballot(word != 0ull) == 0ull;
  if (lane == 0) p.cls[tile] = (unsigned char)(empty ? kClsEmpty : (full ? kClsFull : kClsPart));
  if (!full && !empty) p.ws_bits[tile * 64 + lane] = word;
}

constexpr int kMaxDevices = 64;
unsigned char* g_scratch_ptr[kMaxDevices] = {nullptr};

int static_scratch(unsigned char** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return STOF_ERR_LAUNCH;
  unsigned char* cached = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_RELAXED);
  if (!cached) {   // (two threads that both find the slot empty store the same address)
    void* ptr = nullptr;
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return STOF_ERR_LAUNCH;
    cached = static_cast<unsigned char*>(ptr);
    __atomic_store_n(&g_scratch_ptr[dev], cached, __ATOMIC_RELAXED);
  }
  *out = cached;
  return STOF_OK;
}

bool block_ok(int b) { return b == 16 || b == 32 || b == 64 || b == 128; }

// Workspace layout: class bytes | bit rows (64 x 64 blocks only) | non-zero count per tile (2 bytes) | total (8 bytes + 8 spare)
int64_t ws_cnt_offset(int64_t tiles, int block_m, int block_n) {
  return (tiles + 255) / 256 * 256 + ((block_m == 64 && block_n == 64) ? tiles * 64 * 8 : 0);
}

int check_common(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n) {
  if (!mask) return STOF_ERR_NULL_POINTER;
  if (elem_bytes != 2 && elem_bytes != 4) return STOF_ERR_UNSUPPORTED;
  if (!block_ok(block_m) || !block_ok(block_n)) return STOF_ERR_UNSUPPORTED;
  if (seq_len <= 0 || seq_len % block_m != 0 || seq_len % block_n != 0 || ld < seq_len) return STOF_ERR_BAD_SHAPE;
  if (!stof_aligned16(mask) || (ld * elem_bytes) % 16 != 0) return STOF_ERR_MISALIGNED;
  return STOF_OK;
}

int build(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
          int32_t* frp, int32_t* fci, int32_t* prp, int32_t* pci, int32_t* lrp, int32_t* lci,
          uint64_t* part_bitmask, int32_t* counts, int64_t cap_full, int64_t cap_part, int64_t cap_load,
          unsigned char* cls, uint64_t* ws_bits, unsigned short* cnt, long long* nnz, hipStream_t stream) {
  LutParams p;
  p.cnt = cnt; p.nnz = nnz;
  p.mask = mask; p.ld = ld; p.S = seq_len; p.bm = block_m; p.bn = block_n;
  p.nQ = seq_len / block_m; p.nK = seq_len / block_n;
  p.cls = cls; p.ws_bits = (block_m == 64 && block_n == 64 && part_bitmask) ? ws_bits : nullptr;
  p.frp = frp; p.fci = fci; p.prp = prp; p.pci = pci; p.lrp = lrp; p.lci = lci;
  p.pbits = p.ws_bits ? part_bitmask : nullptr; p.counts = counts;
  p.cap_full = cap_full; p.cap_part = cap_part; p.cap_load = cap_load;
  const int64_t tiles = (int64_t)p.nQ * p.nK;
  const dim3 grid1((unsigned)((tiles + 3) / 4)), block(256);
  if (elem_bytes == 2) hipLaunchKernelGGL(lut_classify_kernel<half_t>, grid1, block, 0, stream, p);
  else hipLaunchKernelGGL(lut_classify_kernel<float>, grid1, block, 0, stream, p);
  hipLaunchKernelGGL(lut_compact_kernel, dim3((unsigned)p.nQ), block, 0, stream, p);
  return stof_check_launch();
}

int check_outputs(const int32_t* frp, const int32_t* fci, const int32_t* prp, const int32_t* pci,
                  const int32_t* lrp, const int32_t* lci, const uint64_t* part_bitmask, int block_m, int block_n,
                  int64_t cap_full, int64_t cap_part, int64_t cap_load) {
  if (!frp || !prp || !lrp) return STOF_ERR_NULL_POINTER;
  if (cap_full < 0 || cap_part < 0 || cap_load < 0) return STOF_ERR_BAD_SHAPE;
  if ((cap_full > 0 && !fci) || (cap_part > 0 && !pci) || (cap_load > 0 && !lci)) return STOF_ERR_NULL_POINTER;
  if (part_bitmask && (block_m != 64 || block_n != 64)) return STOF_ERR_UNSUPPORTED;
  return STOF_OK;
}

}  // namespace

extern "C" int64_t stof_build_lut_workspace_bytes(int seq_len, int block_m, int block_n) {
  if (seq_len <= 0 || !block_ok(block_m) || !block_ok(block_n) || seq_len % block_m || seq_len % block_n) return STOF_ERR_BAD_SHAPE;
  const int64_t tiles = (int64_t)(seq_len / block_m) * (seq_len / block_n);
  return ws_cnt_offset(tiles, block_m, block_n) + (tiles * 2 + 15) / 16 * 16 + 16;
}

extern "C" int64_t stof_build_lut_nnz_offset(int seq_len, int block_m, int block_n) {
  const int64_t total = stof_build_lut_workspace_bytes(seq_len, block_m, block_n);
  return total < 0 ? total : total - 16;
}

extern "C" int stof_build_lut(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
                              int32_t* full_row_ptr, int32_t* full_col_idx,
                              int32_t* part_row_ptr, int32_t* part_col_idx,
                              int32_t* load_row_ptr, int32_t* load_col_idx,
                              uint64_t* part_bitmask, int32_t* counts,
                              int64_t cap_full, int64_t cap_part, int64_t cap_load,
                              void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = check_common(mask, elem_bytes, ld, seq_len, block_m, block_n);
  if (rc != STOF_OK) return rc;
  rc = check_outputs(full_row_ptr, full_col_idx, part_row_ptr, part_col_idx, load_row_ptr, load_col_idx,
                     part_bitmask, block_m, block_n, cap_full, cap_part, cap_load);
  if (rc != STOF_OK) return rc;
  if (!workspace) return STOF_ERR_NULL_POINTER;
  if (workspace_bytes < stof_build_lut_workspace_bytes(seq_len, block_m, block_n)) return STOF_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(workspace) & 7) != 0) return STOF_ERR_MISALIGNED;
  const int64_t tiles = (int64_t)(seq_len / block_m) * (seq_len / block_n);
  unsigned char* cls = static_cast<unsigned char*>(workspace);
  uint64_t* bits = reinterpret_cast<uint64_t*>(cls + (tiles + 255) / 256 * 256);
  unsigned short* cnt = reinterpret_cast<unsigned short*>(cls + ws_cnt_offset(tiles, block_m, block_n));
  long long* nnz = reinterpret_cast<long long*>(cls + stof_build_lut_nnz_offset(seq_len, block_m, block_n));
  return build(mask, elem_bytes, ld, seq_len, block_m, block_n, full_row_ptr, full_col_idx, part_row_ptr, part_col_idx,
               load_row_ptr, load_col_idx, part_bitmask, counts, cap_full, cap_part, cap_load, cls, bits, cnt, nnz, (hipStream_t)stream);
}

extern "C" int stof_retile_lut(const int32_t* full_row_ptr, const int32_t* full_col_idx,
                               const int32_t* part_row_ptr, const int32_t* part_col_idx, const void* part_block_mask,
                               int block_m, int block_n, int seq_len,
                               int32_t* out_full_row_ptr, int32_t* out_full_col_idx,
                               int32_t* out_part_row_ptr, int32_t* out_part_col_idx,
                               int32_t* out_load_row_ptr, int32_t* out_load_col_idx,
                               uint64_t* out_part_bitmask, int32_t* counts,
                               int64_t cap_full, int64_t cap_part, int64_t cap_load,
                               void* workspace, int64_t workspace_bytes, void* stream) {
  if (!full_row_ptr || !part_row_ptr) return STOF_ERR_NULL_POINTER;
  if (!block_ok(block_m) || !block_ok(block_n)) return STOF_ERR_UNSUPPORTED;
  if (seq_len <= 0 || seq_len % 64 != 0 || seq_len % block_m != 0 || seq_len % block_n != 0) return STOF_ERR_BAD_SHAPE;
  if (part_block_mask && !stof_aligned16(part_block_mask)) return STOF_ERR_MISALIGNED;
  int rc = check_outputs(out_full_row_ptr, out_full_col_idx, out_part_row_ptr, out_part_col_idx, out_load_row_ptr, out_load_col_idx,
                         out_part_bitmask, 64, 64, cap_full, cap_part, cap_load);
  if (rc != STOF_OK) return rc;
  if (!workspace || !out_part_bitmask) return STOF_ERR_NULL_POINTER;
  if (workspace_bytes < stof_build_lut_workspace_bytes(seq_len, 64, 64)) return STOF_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(workspace) & 7) != 0) return STOF_ERR_MISALIGNED;
  const int n64 = seq_len / 64;
  const int64_t tiles = (int64_t)n64 * n64;
  RetileParams r;
  r.frp = full_row_ptr; r.fci = full_col_idx; r.prp = part_row_ptr; r.pci = part_col_idx; r.pbm = (const half_t*)part_block_mask;
  r.bm = block_m; r.bn = block_n; r.n64 = n64;
  r.cls = static_cast<unsigned char*>(workspace);
  r.ws_bits = reinterpret_cast<uint64_t*>(r.cls + (tiles + 255) / 256 * 256);
  hipLaunchKernelGGL(lut_retile_kernel, dim3((unsigned)((tiles + 3) / 4)), dim3(256), 0, (hipStream_t)stream, r);
  LutParams p;
  p.mask = nullptr; p.ld = 0; p.S = seq_len; p.bm = 64; p.bn = 64; p.nQ = n64; p.nK = n64;
  p.cls = r.cls; p.ws_bits = r.ws_bits; p.cnt = nullptr; p.nnz = nullptr;
  p.frp = out_full_row_ptr; p.fci = out_full_col_idx; p.prp = out_part_row_ptr; p.pci = out_part_col_idx;
  p.lrp = out_load_row_ptr; p.lci = out_load_col_idx; p.pbits = out_part_bitmask; p.counts = counts;
  p.cap_full = cap_full; p.cap_part = cap_part; p.cap_load = cap_load;
  hipLaunchKernelGGL(lut_compact_kernel, dim3((unsigned)n64), dim3(256), 0, (hipStream_t)stream, p);
  return stof_check_launch();
}

extern "C" int64_t stof_build_lut_static_max_tiles(void) { return kStaticMaxTiles; }

extern "C" int stof_build_lut_static(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
                                     int32_t* full_row_ptr, int32_t* full_col_idx,
                                     int32_t* part_row_ptr, int32_t* part_col_idx,
                                     int32_t* load_row_ptr, int32_t* load_col_idx,
                                     uint64_t* part_bitmask, int32_t* counts,
                                     int64_t cap_full, int64_t cap_part, int64_t cap_load, void* stream) {
  int rc = check_common(mask, elem_bytes, ld, seq_len, block_m, block_n);
  if (rc != STOF_OK) return rc;
  rc = check_outputs(full_row_ptr, full_col_idx, part_row_ptr, part_col_idx, load_row_ptr, load_col_idx,
                     part_bitmask, block_m, block_n, cap_full, cap_part, cap_load);
  if (rc != STOF_OK) return rc;
  const int64_t tiles = (int64_t)(seq_len / block_m) * (seq_len / block_n);
  if (tiles > kStaticMaxTiles) return STOF_ERR_TOO_LARGE;   // beyond the fixed scratch: use stof_build_lut with a workspace
  unsigned char* ptr = nullptr;   // this device's copy of the scratch array
  rc = static_scratch(&ptr);
  if (rc != STOF_OK) return rc;
  return build(mask, elem_bytes, ld, seq_len, block_m, block_n, full_row_ptr, full_col_idx, part_row_ptr, part_col_idx,
               load_row_ptr, load_col_idx, part_bitmask, counts, cap_full, cap_part, cap_load,
               ptr, reinterpret_cast<uint64_t*>(ptr + kClsBytesStatic),
               reinterpret_cast<unsigned short*>(ptr + kClsBytesStatic + kBitsBytesStatic),
               reinterpret_cast<long long*>(ptr + kClsBytesStatic + kBitsBytesStatic + kStaticMaxTiles * 2), (hipStream_t)stream);
}

extern "C" int stof_lut_additive_blocks(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
                                        const int32_t* part_row_ptr, const int32_t* part_col_idx, int64_t n_part,
                                        void* part_block_mask, void* stream) {
  int rc = check_common(mask, elem_bytes, ld, seq_len, block_m, block_n);
  if (rc != STOF_OK) return rc;
  if (n_part < 0 || n_part > ((int64_t)1 << 30)) return STOF_ERR_BAD_SHAPE;
  if (n_part == 0) return STOF_OK;
  if (!part_row_ptr || !part_col_idx || !part_block_mask) return STOF_ERR_NULL_POINTER;
  const int nQ = seq_len / block_m;
  if (elem_bytes == 2)
    hipLaunchKernelGGL(lut_additive_blocks_kernel<half_t>, dim3((unsigned)n_part), dim3(256), 0, (hipStream_t)stream,
                       mask, ld, block_m, block_n, nQ, part_row_ptr, part_col_idx, (half_t*)part_block_mask);
  else
    hipLaunchKernelGGL(lut_additive_blocks_kernel<float>, dim3((unsigned)n_part), dim3(256), 0, (hipStream_t)stream,
                       mask, ld, block_m, block_n, nQ, part_row_ptr, part_col_idx, (half_t*)part_block_mask);
  return stof_check_launch();
}
