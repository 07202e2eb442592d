// Block-masked multi-head attention for gfx950 (MI355X), head size 64, 64x64 LUT blocks.
//
// Replaces the 20 WMMA kernels + dispatcher of the reference
// (src/ops/src/block_attn_mask_cuda.cu:269-6322) with one kernel designed around the
// CDNA4 wavefront:
//
//  * a wave keeps 32 queries in registers; S, P and O never touch LDS.  A workgroup of four
//    64-lane wavefronts runs in one of two forms.  Large grids: it owns TWO adjacent 64-row
//    query blocks (two LUT rows) whose key-block lists are merged on the fly; a key block
//    wanted by both rows is brought into LDS once and used by all four waves, one wanted by a
//    single row is skipped by the other row's waves.  This halves the L2 -> LDS traffic per
//    unit of MFMA work.  Small grids: it owns ONE query block and the two wave pairs take
//    the two 32-key halves of every tile, so the chain of key blocks of a long row, which
//    sets the run time there, takes half as long; partial results are merged through LDS;
//  * K/V tiles travel HBM/L2 -> LDS with the asynchronous direct-to-LDS loads
//    (global_load_lds_dwordx4), double buffered: the loads of block t+1 are issued before
//    the math of block t, no VGPRs are used for staging and one barrier per block suffices;
//  * scores are produced TRANSPOSED, S^T = K . Q^T, with v_mfma_f32_32x32x16_f16.  In the
//    32x32 accumulator layout a lane holds 32 keys of ONE query (lane & 31), so the
//    online-softmax state (running max, running sum, rescale factor) is one scalar per
//    lane, the row reduction is a register loop plus one v_permlane32_swap, and the
//    probabilities already sit in the register layout the second product
//    O^T = V^T . P^T wants for its B operand;
//  * V stays row-major in LDS; the A operand of the second product (key index contiguous
//    per lane) is formed by the transposing LDS read ds_read_b64_tr_b16;
//  * LDS tiles are unpadded (the DMA writes 1 KB contiguous per instruction); a 16-byte
//    chunk XOR swizzle applied on the global-address side keeps both the 16-byte K
//    fragment reads and the transposing V reads free of bank conflicts;
//  * masks: full tiles run mask-free, partial tiles test one bit per element from a
//    64-bit row mask (512 B per tile instead of the reference's 8 KB additive fp16 tile),
//    empty tiles are never visited; the LUT row is fetched once into registers;
//  * workgroup ids are remapped so that all query blocks of one (batch, head) run on one
//    XCD (K/V stay in that XCD's L2), and the groups of an XCD are taken in descending order
//    of LUT row length, ranked inside the kernel, and dealt evenly over its compute units;
//    at every step a wave's issue priority follows the number of key blocks it has left.
#include "stof_common.h"

namespace {

constexpr int kD = 64;        // head size
constexpr int kBM = 64;       // query rows per block
constexpr int kBN = 64;       // keys per block
constexpr int kTile = kBN * kD * 2;   // bytes of one K or V tile in LDS (8 KB, unpadded)
constexpr float kLazy = 8.0f;         // log2 slack before the running max is raised
constexpr int kPrioStep = 6;          // key blocks of remaining chain per issue-priority level

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) short4_t lds_short4;
typedef __attribute__((address_space(1))) const void gptr_t;

struct AttnParams {
  const half_t* q; const half_t* k; const half_t* v; half_t* out;
  const int32_t* prp; const int32_t* pci; const uint64_t* pbits;
  const int32_t* lrp; const int32_t* lci;
  int64_t qs[3], ks[3], vs[3], os[3];
  int64_t lut_bs;
  int B, S, H, nQ, nP;   // nP = query-block pairs per (batch, head)
  int total, chunk;
  int balance, cus_per_xcd;   // balance != 0: groups are dealt to compute units by row length (see balanced_group)
  float c;  // softmax_scale * log2(e)
  // row-wise front-ends (KIND != 0): key blocks come from index arithmetic, not from a LUT
  const uint64_t* row_bits; int words; int causal; int band;
};

enum { kKindLut = 0, kKindPred = 1, kKindBits = 2 };

__device__ __forceinline__ floatx16 mfma32(half8_t a, half8_t b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// max / sum of a value with its partner lane (lane ^ 32).  v_permlane32_swap(x, x) leaves
// {own, partner} in some order in its two results for either half of the wave.
__device__ __forceinline__ float pair_max(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}

// 16-byte-chunk swizzle of a tile row: chunk c of row r is stored at chunk position
// c ^ swz(r).  swz is a bijection of row bits (1,2,3) onto chunk bits (2,0,1).
__device__ __forceinline__ int swz(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

// Extents of one LUT row (the key blocks of one 64-row query block).  LOAD is the union of
// FULL and PART with ascending key-block indices (get_sparse_storage builds it so), hence an
// entry is partial iff its key block is in the row's PART list, and the PART slot of a block
// is its rank in that list.
struct RowList {
  int t0, n, p0, np;   // KIND LUT: first LOAD entry, LOAD count, first PART entry, PART count
  int ptr, pptr;       // LOAD / PART entries already handed out to earlier 64-column windows
  int lo, hi;          // KIND != LUT: the contiguous key-block range [lo, hi]
};

// Row pointers of a group's rows when the caller of attn_group has them in registers already.
template <int ROWS> struct RowPtrs {
  int t0[ROWS], n[ROWS], p0[ROWS], np[ROWS];
  bool valid;
};

// ROWS = query blocks per workgroup, KS = key split.  Launched as <2, 1> (four waves: two query
// blocks x two 32-query halves, every wave sees all 64 keys of a tile) or <1, 2> (four waves
// on ONE query block: two 32-query halves x two 32-key halves of every tile, partial results
// merged through LDS at the end).  The second form halves the work of a wave per key block,
// so the chain of key blocks of a long LUT row finishes in half the time; it is used for
// small grids, where that chain and not throughput sets the run time.
template <int KIND, int ROWS, int KS, bool PIPE = false>
__device__ __forceinline__ void attn_group(const AttnParams& p, const int bh, const int pair, const RowPtrs<ROWS>& pre,
                                           unsigned char* k_lds0, unsigned char* k_lds1,
                                           unsigned char* v_lds0, unsigned char* v_lds1) {
  static_assert(KS == 1 || ROWS == 1, "the key split serves a single query block");
  static_assert(!PIPE || KS == 1, "the software-pipelined loop keeps all 64 keys of a tile in one wave");
  constexpr int kDma = 4 / (ROWS * KS);   // direct-to-LDS instructions per wave and operand tile (8 per tile)
  constexpr int kMT = 2 / KS;             // 32-key sub-tiles of a key block handled by one wave

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31;
  const int g = lane >> 5;
  const int rsel = KS == 1 ? wave >> 1 : 0;   // which of the group's query blocks this wave serves
  const int half = wave & 1;                  // which 32 queries of that block
  const int mt0 = KS == 1 ? 0 : wave >> 1;    // first 32-key sub-tile of this wave

  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int qi = ROWS * pair + rsel;               // this wave's query block
  const bool q_valid = qi < p.nQ;                  // block count not a multiple of ROWS: the last group is short

  const int64_t qrow0 = (int64_t)qi * kBM + 32 * half;
  const half_t* qb = p.q + b * p.qs[0] + h * p.qs[1] + qrow0 * p.qs[2];
  const half_t* kb = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vb = p.v + b * p.vs[0] + h * p.vs[1];
  half_t* ob = p.out + b * p.os[0] + h * p.os[1] + qrow0 * p.os[2];

  // ---- the ROWS rows of the group; every wave walks the same merged sequence of key blocks
  const int64_t lo = (int64_t)b * p.lut_bs;
  RowList row[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int qr = ROWS * pair + r;
    row[r].t0 = row[r].n = row[r].p0 = row[r].np = row[r].ptr = row[r].pptr = 0;
    row[r].lo = 0; row[r].hi = -1;
    if (qr < p.nQ) {
      if (KIND == kKindLut) {
        if (pre.valid) {   // the placement code has read the row pointers already
          row[r].t0 = pre.t0[r]; row[r].n = pre.n[r]; row[r].p0 = pre.p0[r]; row[r].np = pre.np[r];
        } else {
          row[r].t0 = __builtin_amdgcn_readfirstlane(p.lrp[lo + qr]);
          row[r].n = __builtin_amdgcn_readfirstlane(p.lrp[lo + qr + 1]) - row[r].t0;
          row[r].p0 = __builtin_amdgcn_readfirstlane(p.prp[lo + qr]);
          row[r].np = __builtin_amdgcn_readfirstlane(p.prp[lo + qr + 1]) - row[r].p0;
        }
      } else {
        // keys allowed for some query of block qr: (64qr - band, 64qr + 63] when sliding,
        // up to the diagonal block when causal, else every block
        row[r].hi = p.causal ? qr : p.nQ - 1;
        const int first_key = (KIND == kKindPred && p.band > 0) ? 64 * qr - p.band + 1 : 0;
        row[r].lo = first_key > 0 ? first_key / 64 : 0;
      }
    }
  }

  // LUT entries of the current window of 64 key blocks: lane l holds entry ptr + l of each row's
  // LOAD list and of this wave's PART list.  Every list read of a window goes out before the
  // first is waited for, and window 0 is requested here, AHEAD of the Q loads: the memory
  // counter retires in order, so the wait for these (L2-resident) entries does not also wait
  // for Q (HBM), whose latency then overlaps the walk set-up and the first K/V loads.
  int win_e[ROWS], win_pe = 0x7fffffff;
  auto fetch_window = [&]() {
    win_pe = 0x7fffffff;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      win_e[r] = 0x7fffffff;
      if (KIND == kKindLut) {
        if (row[r].ptr + lane < row[r].n) win_e[r] = p.lci[row[r].t0 + row[r].ptr + lane];
        if (r == rsel && row[r].pptr + lane < row[r].np) win_pe = p.pci[row[r].p0 + row[r].pptr + lane];
      }
    }
  };
  fetch_window();
  __builtin_amdgcn_sched_barrier(0);

  // Q^T as the B operand: lane (n = query j32, k-group g) holds 8 consecutive d per k-step.
  // (A query block past the end - odd block count, last group - reads the last real block
  // instead: its row lists are empty and nothing of it is stored.)
  half8_t qf[4];
  {
    const half_t* qsrc = q_valid ? qb : qb - (int64_t)kBM * p.qs[2];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) qf[ks] = *reinterpret_cast<const half8_t*>(qsrc + (int64_t)j32 * p.qs[2] + 16 * ks + 8 * g);
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- per-lane constants of the data movement
  // DMA: a tile is 8 instructions of 1 KB (8 rows of 128 B); wave w issues instructions
  // kDma*w .. kDma*w + kDma - 1 for K and for V.  Lane l lands at (row 8*ii + l/8, chunk
  // position l%8) and therefore fetches global chunk (l%8) ^ swz(row).
  // Per-lane BYTE offsets inside a tile, unsigned 32-bit: the load then takes the tile's
  // wave-uniform base in scalar registers and this as its vector offset.
  uint32_t k_src[kDma], v_src[kDma];
#pragma unroll
  for (int i = 0; i < kDma; ++i) {
    const int trow = 8 * (kDma * wave + i) + (lane >> 3);
    const int chunk = (lane & 7) ^ swz(trow);
    k_src[i] = (uint32_t)trow * (uint32_t)(p.ks[2] * 2) + 16 * chunk;
    v_src[i] = (uint32_t)trow * (uint32_t)(p.vs[2] * 2) + 16 * chunk;
  }
  // K fragment (A operand of S^T): row = key 32*mt + j32, chunk 2*ks + g.
  int k_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) k_rd[ks] = j32 * 128 + (((2 * ks + g) ^ swz(j32)) << 4);
  // V fragment (A operand of O^T) through the transposing read.  Within a 16-lane block,
  // lane j supplies the address of key row (j >> 2) at channel offset 4*(j & 3) and receives
  // the four keys of channel (block base + j).  Block = lane >> 4: k-group g = block >> 1,
  // channel half = block & 1.  Keys of k-step (mt, s2), half hh: 32mt + 16s2 + 8hh + 4g + c.
  int v_rd[2][2];
  {
    const int j = lane & 15, dh = (lane >> 4) & 1;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int vrow = 8 * hh + 4 * g + (j >> 2);
        const int chunk = 4 * dt + 2 * dh + ((j >> 1) & 1);
        v_rd[dt][hh] = vrow * 128 + ((chunk ^ swz(vrow)) << 4) + 8 * (j & 1);
      }
  }

  // Key blocks this wave still has to visit (the longer of the group's rows: a lower bound of
  // the merged walk).  It sets the wave's issue priority at every step - see step().
  int steps_left = 0;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) steps_left = max(steps_left, KIND == kKindLut ? row[r].n : row[r].hi - row[r].lo + 1);

  floatx16 oacc[2];   // [d tile]: O^T for this wave's 32 queries
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;

  auto issue_tile = [&](int col, lds_byte* kdst, lds_byte* vdst) {
    const char* kt = reinterpret_cast<const char*>(kb + (int64_t)col * kBN * p.ks[2]);
    const char* vt = reinterpret_cast<const char*>(vb + (int64_t)col * kBN * p.vs[2]);
    lds_byte* kd = kdst + (kDma * wave) * 1024;
    lds_byte* vd = vdst + (kDma * wave) * 1024;
#pragma unroll
    for (int i = 0; i < kDma; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t*)(kt + k_src[i]), (__attribute__((address_space(3))) void*)(kd + i * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < kDma; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t*)(vt + v_src[i]), (__attribute__((address_space(3))) void*)(vd + i * 1024), 16, 0, 0);
  };

  // ---- merged walk over the group's rows, wave-uniform and identical in every wave.
  // Key blocks are handled in windows of 64: per window each row's active blocks form a
  // 64-bit set, the union of the sets is walked with find-first-set, a block listed by
  // several rows is loaded once, and the bitmask slot of a partial block is the PART list
  // offset of the window plus the population count of the PART set below the block.
  struct Step { int col; int mine; int slot; bool valid; };
  const int n_win = (p.nQ + 63) >> 6;
  int win = 0;   // window 0 is consumed right below, outside the walk's loop
  uint64_t set_union = 0, set_mine = 0, set_part = 0;
  int part_base = 0;
  auto consume_window = [&](int w) {
    set_union = 0; set_mine = 0; set_part = 0;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      uint64_t m = 0;
      if (KIND == kKindLut) {
        const int cnt = __builtin_popcountll(__ballot(win_e[r] < 64 * (w + 1)));
        for (int j = 0; j < cnt; ++j) m |= 1ull << (__builtin_amdgcn_readlane(win_e[r], j) - 64 * w);
        row[r].ptr += cnt;
        if (r == rsel) {
          const int pcnt = __builtin_popcountll(__ballot(win_pe < 64 * (w + 1)));
          for (int j = 0; j < pcnt; ++j) set_part |= 1ull << (__builtin_amdgcn_readlane(win_pe, j) - 64 * w);
          part_base = row[r].p0 + row[r].pptr;
          row[r].pptr += pcnt;
        }
      } else {
        const int a = max(row[r].lo, 64 * w), z = min(row[r].hi, 64 * w + 63);
        if (a <= z) m = ((z - a == 63) ? ~0ull : ((1ull << (z - a + 1)) - 1)) << (a - 64 * w);
      }
      set_union |= m;
      if (r == rsel) set_mine = m;
    }
  };
  consume_window(0);
  auto next_step = [&]() -> Step {
    Step s; s.col = 0; s.mine = 0; s.slot = -1; s.valid = false;
    while (set_union == 0) {
      if (++win >= n_win) return s;
      fetch_window();
      consume_window(win);
    }
    const int bit = __builtin_ctzll(set_union);
    set_union &= set_union - 1;
    s.valid = true;
    s.col = 64 * win + bit;
    s.mine = (int)((set_mine >> bit) & 1);
    if (KIND == kKindLut && s.mine && ((set_part >> bit) & 1))
      s.slot = part_base + __builtin_popcountll(set_part & ((1ull << bit) - 1));
    return s;
  };

  if constexpr (PIPE) {
    // ---- software-pipelined main loop.
    // Iteration i holds three tiles of the wave's chain at once: the scores of tile i+1 are
    // produced (S = K Q^T, 8 MFMA), the probabilities of tile i are formed from the scores made
    // one iteration ago (exp2, convert, row sum: vector ALU only) and the probabilities of tile
    // i-1 go into O (O += V^T P^T, 8 MFMA).  The three are independent of one another, so inside
    // ONE wave every MFMA is followed by vector-ALU work that does not wait for it: the matrix
    // pipeline and the vector ALU run side by side.  (Across waves they overlap badly: an MFMA
    // that waits for the pipeline holds the SIMD's issue slot.)
    //
    // Running max: the fast path takes the max as it stands and only verifies, from the row sums
    // it needs anyway, that no probability left the fp16 range; if one did (or a lane has not
    // seen a key yet, or a tile needs an element mask, or a neighbour tile is not this wave's),
    // the iteration runs the general path below: exact online softmax with max search and
    // rescale, one piece after the other.  O holds tile i-1 by then, so the rescale is the usual one.
    //
    // LDS: K is fetched two tiles ahead of V (iteration i issues K(i+2) and V(i), reads K(i+1) and
    // V(i-1)); with two buffers each, an iteration reads one buffer pair and fills the other.
    struct Tile { Step st; bool mask; };
    auto dma_k = [&](int col, lds_byte* kdst) {
      const char* kt = reinterpret_cast<const char*>(kb + (int64_t)col * kBN * p.ks[2]);
      lds_byte* kd = kdst + (kDma * wave) * 1024;
#pragma unroll
      for (int i = 0; i < kDma; ++i)
        __builtin_amdgcn_global_load_lds((gptr_t*)(kt + k_src[i]), (__attribute__((address_space(3))) void*)(kd + i * 1024), 16, 0, 0);
    };
    auto dma_v = [&](int col, lds_byte* vdst) {
      const char* vt = reinterpret_cast<const char*>(vb + (int64_t)col * kBN * p.vs[2]);
      lds_byte* vd = vdst + (kDma * wave) * 1024;
#pragma unroll
      for (int i = 0; i < kDma; ++i)
        __builtin_amdgcn_global_load_lds((gptr_t*)(vt + v_src[i]), (__attribute__((address_space(3))) void*)(vd + i * 1024), 16, 0, 0);
    };
    // element-mask word of this lane's query for a tile (requested when the tile enters the queue)
    auto request_bits = [&](const Step& st) -> uint64_t {
      uint64_t bits = ~0ull;
      if (KIND == kKindLut) {
        if (st.valid && st.slot >= 0) bits = p.pbits[(int64_t)st.slot * kBM + 32 * half + j32];
      } else if (KIND == kKindBits) {
        if (st.valid && st.mine) bits = p.row_bits[(qrow0 + j32) * p.words + st.col];
      }
      return bits;
    };
    // whether the tile needs its element mask (wave-uniform); the index predicates of the
    // row-wise front-ends are folded into the bit row; a tile that allows nothing is dropped
    auto settle_mask = [&](Tile& t, uint64_t& bits) {
      t.mask = false;
      if (!t.st.valid || !t.st.mine) return;
      if (KIND == kKindLut) { t.mask = t.st.slot >= 0; return; }
      const int qmin = (int)qrow0, qmax = qmin + 31, kmin = t.st.col * kBN, kmax = kmin + kBN - 1;
      const bool range_full = (!p.causal || kmax <= qmin) && (!(KIND == kKindPred && p.band > 0) || kmin > qmax - p.band);
      if (KIND == kKindBits) {
        if (!__any(bits != 0ull)) { t.st.mine = 0; return; }
        t.mask = !range_full || __any(bits != ~0ull);
      } else {
        t.mask = !range_full;
      }
      if (t.mask) {
        const int qg = qmin + j32;
        if (p.causal) { const int nk = qg - kmin + 1; bits &= nk >= 64 ? ~0ull : (nk <= 0 ? 0ull : ((1ull << nk) - 1)); }
        if (KIND == kKindPred && p.band > 0) {
          const int first = qg - p.band + 1 - kmin;
          bits &= first <= 0 ? ~0ull : (first >= 64 ? 0ull : ~((1ull << first) - 1));
        }
      }
    };
    // S^T = K . Q^T into s (see the accumulator layout at the non-pipelined step)
    auto qk_product = [&](const lds_byte* kt, floatx16 (&s)[2]) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const half8_t a = *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(kt + mt * 4096 + k_rd[ks]);
          s[mt] = mfma32(a, qf[ks], s[mt]);
        }
    };
    auto init_scores = [&](floatx16 (&s)[2], bool masked, uint64_t bits) {
      if (masked) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const uint32_t nw = ~((uint32_t)(bits >> (32 * mt)) >> (4 * g));   // bit set = key masked
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            int all;   // -1 if masked, else 0
            asm("v_bfe_i32 %0, %1, %2, 1" : "=v"(all) : "v"(nw), "n"(8 * (r >> 2) + (r & 3)));
            s[mt][r] = __builtin_bit_cast(float, (uint32_t)all & 0xFF800000u);
          }
        }
      } else {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[mt][r] = 0.f;
      }
    };
    // O^T += V^T . P^T
    auto pv_product = [&](const lds_byte* vt, const half8_t (&pf)[2][2]) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int dt = 0; dt < 2; ++dt) {
            const lds_byte* vp = vt + (32 * mt + 16 * s2) * 128;
            const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vp + v_rd[dt][0]));
            const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vp + v_rd[dt][1]));
            const half8_t a = __builtin_bit_cast(half8_t, (short8_t)__builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
            oacc[dt] = mfma32(a, pf[mt][s2], oacc[dt]);
          }
    };
    bool warm = false;   // every lane of the wave has a finite running max
    float mc = 0.f;      // running max * c, the constant the fast softmax subtracts
    // exact online softmax of one tile (max search, lazy raise, rescale of O and of the sum)
    auto softmax_exact = [&](const floatx16 (&s)[2], half8_t (&pf)[2][2]) {
      float mx = s[0][0];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[mt][r]);
      mx = pair_max(mx);
      const float m_new = (mx * p.c > m_run * p.c + kLazy || m_run == -INFINITY) ? mx : m_run;
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_sub) * p.c);
      mc = m_sub * p.c;
      float lsum = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][r], p.c, -mc));
          const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][r + 1], p.c, -mc));
          const half2_t e2 = {(half_t)e0, (half_t)e1};
          pf[mt][r >> 3][r & 7] = e2[0];
          pf[mt][r >> 3][(r & 7) + 1] = e2[1];
          lsum += e0 + e1;
        }
      l_run = l_run * alpha + lsum;
      m_run = m_new;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
      }
      warm = !__any(m_run == -INFINITY);
    };
    // Fast softmax: the max is taken as it stands.  The row sum is formed from the fp16
    // probabilities themselves (the values the second product uses) by a tree of packed adds,
    // folded to fp32 once; a probability beyond the fp16 range shows up in it as inf or as a
    // large sum, which the caller tests before it commits the tile.
    auto softmax_fast = [&](const floatx16 (&s)[2], half8_t (&pf)[2][2]) -> float {
      half2_t acc[16];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][r], p.c, -mc));
          const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mt][r + 1], p.c, -mc));
          const half2_t e2 = {(half_t)e0, (half_t)e1};
          pf[mt][r >> 3][r & 7] = e2[0];
          pf[mt][r >> 3][(r & 7) + 1] = e2[1];
          acc[8 * mt + (r >> 1)] = e2;
        }
#pragma unroll
      for (int w = 8; w > 0; w >>= 1)
#pragma unroll
        for (int i = 0; i < w; ++i) acc[i] = acc[i] + acc[i + w];
      return (float)acc[0][0] + (float)acc[0][1];
    };
    constexpr float kSumLimit = 16384.f;   // 32 probabilities of at most 2^kLazy sum to 2^13

    Tile t0, t1, t2, t3;   // tiles i-1 (PV), i (softmax), i+1 (QK^T), i+2 (loads)
    t0.st.valid = t1.st.valid = t2.st.valid = false;
    t0.st.mine = t1.st.mine = t2.st.mine = 0;
    t0.st.col = t1.st.col = t2.st.col = 0; t0.st.slot = t1.st.slot = t2.st.slot = -1;
    t0.mask = t1.mask = t2.mask = t3.mask = false;
    t3.st = next_step();
    uint64_t bits2 = ~0ull;          // mask word of tile t2
    floatx16 sA[2], sB[2];
    half8_t pA[2][2], pB[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) { sA[mt][r] = 0.f; sB[mt][r] = 0.f; }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int e = 0; e < 8; ++e) { pA[mt][s2][e] = (half_t)0.f; pB[mt][s2][e] = (half_t)0.f; }
    }

    // One iteration: reads the buffer pair (kr, vr), fills (kw, vw); scores s_in -> probabilities
    // p_out, scores of the next tile -> s_out, probabilities p_in -> O.
    auto iteration = [&](const lds_byte* kr, const lds_byte* vr, lds_byte* kw, lds_byte* vw,
                         floatx16 (&s_in)[2], floatx16 (&s_out)[2], half8_t (&p_in)[2][2], half8_t (&p_out)[2][2]) {
      {
        const int left = steps_left--;
        if (left >= 3 * kPrioStep) __builtin_amdgcn_s_setprio(3);
        else if (left >= 2 * kPrioStep) __builtin_amdgcn_s_setprio(2);
        else if (left >= kPrioStep) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): K(i+1), V(i-1) and the mask word of tile i+1 have landed
      __syncthreads();
      if (t3.st.valid) dma_k(t3.st.col, kw);
      if (t1.st.valid) dma_v(t1.st.col, vw);
      const uint64_t bits3 = request_bits(t3.st);
      settle_mask(t2, bits2);
      const bool do_pv = t0.st.valid && t0.st.mine, do_sm = t1.st.valid && t1.st.mine, do_qk = t2.st.valid && t2.st.mine;
      if (do_pv && do_sm && do_qk && !t2.mask && warm) {
        init_scores(s_out, false, 0);
        qk_product(kr, s_out);
        const float lsum = softmax_fast(s_in, p_out);
        pv_product(vr, p_in);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // LDS fragment reads of the MFMAs to come
          __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);   // two exp2
          __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);   // scale, convert, sum
        }
        if (__any(!(lsum < kSumLimit))) softmax_exact(s_in, p_out);
        else l_run += lsum;
      } else {
        if (do_qk) { init_scores(s_out, t2.mask, bits2); qk_product(kr, s_out); }
        if (do_pv) pv_product(vr, p_in);
        if (do_sm) softmax_exact(s_in, p_out);
      }
      t0 = t1; t1 = t2; t2 = t3;
      bits2 = bits3;
      t3.st = next_step(); t3.mask = false;
    };

    while (t0.st.valid || t1.st.valid || t2.st.valid || t3.st.valid) {   // single exit
      iteration((const lds_byte*)k_lds1, (const lds_byte*)v_lds1, (lds_byte*)k_lds0, (lds_byte*)v_lds0, sA, sB, pA, pB);
      iteration((const lds_byte*)k_lds0, (const lds_byte*)v_lds0, (lds_byte*)k_lds1, (lds_byte*)v_lds1, sB, sA, pB, pA);
    }
  } else {
    // one key block: kt/vt hold the current tile, the next tile's loads go to kn/vn
    auto step = [&](const Step cur, const Step nxt, const lds_byte* kt, const lds_byte* vt, lds_byte* kn, lds_byte* vn) {
      // The row mask of a partial tile is fetched first so that its latency hides behind
      // the wait below and no register-returning load is pending across the DMA issue.
      // Longest remaining chain first.  Among waves of equal priority a SIMD issues from the
      // oldest, which starves the youngest workgroup of a compute unit until the others are done
      // and leaves it to finish a long chain alone (measured: the last of four equal chains had
      // done 6 of 21 steps when the third finished).  Priority by remaining length makes the
      // chains of a SIMD end together.
      {
        const int left = steps_left--;
        if (left >= 3 * kPrioStep) __builtin_amdgcn_s_setprio(3);
        else if (left >= 2 * kPrioStep) __builtin_amdgcn_s_setprio(2);
        else if (left >= kPrioStep) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
      }
      uint64_t bits = ~0ull;
      if (KIND == kKindLut) {
        if (cur.slot >= 0) bits = p.pbits[(int64_t)cur.slot * kBM + 32 * half + j32];
      } else if (KIND == kKindBits) {
        if (cur.mine) bits = p.row_bits[(qrow0 + j32) * p.words + cur.col];
      }
      // All DMA issued so far (the current tile) has landed for this wave; the barrier makes
      // every wave's share visible and also orders last step's reads of the other buffers
      // before the loads that overwrite them.
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
      __syncthreads();
      if (nxt.valid) issue_tile(nxt.col, kn, vn);
      if (!cur.mine) return;
      // Row-wise front-ends: which elements of this tile may be used.  need_mask is wave-uniform.
      bool need_mask = (KIND == kKindLut) ? (cur.slot >= 0) : false;
      if (KIND != kKindLut) {
        const int qmin = (int)qrow0, qmax = qmin + 31, kmin = cur.col * kBN, kmax = kmin + kBN - 1;
        const bool range_full = (!p.causal || kmax <= qmin) && (!(KIND == kKindPred && p.band > 0) || kmin > qmax - p.band);
        if (KIND == kKindBits) {
          if (!__any(bits != 0ull)) return;            // nothing allowed for these 32 queries
          need_mask = !range_full || __any(bits != ~0ull);
        } else {
          need_mask = !range_full;
        }
        if (need_mask) {
          // fold the index predicates into the bit row: bit t = key kmin + t allowed
          const int qg = qmin + j32;
          if (p.causal) { const int nk = qg - kmin + 1; bits &= nk >= 64 ? ~0ull : (nk <= 0 ? 0ull : ((1ull << nk) - 1)); }
          if (KIND == kKindPred && p.band > 0) {
            const int first = qg - p.band + 1 - kmin;   // keys below this offset are outside the window
            bits &= first <= 0 ? ~0ull : (first >= 64 ? 0ull : ~((1ull << first) - 1));
          }
        }
      }

      // ---- S^T = K . Q^T : sacc[mt][r] = S[query j32][key 32mt + 8(r/4) + 4g + r%4]
      // A partial tile applies its element mask through the accumulator's INITIAL value: 0 where
      // the key is allowed, -inf where it is not (-inf + finite = -inf), two instructions per
      // element (sign-extended one-bit field of the inverted mask word, AND with the bit pattern
      // of -inf) instead of test + compare + select after the product.  The two cases run their
      // own copy of the product so that the unmasked one keeps the constant-zero accumulator input.
      floatx16 sacc[kMT];
      auto s_product = [&]() {
  #pragma unroll
        for (int ks = 0; ks < 4; ++ks)
  #pragma unroll
          for (int mt = 0; mt < kMT; ++mt) {
            const half8_t a = *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(kt + (mt0 + mt) * 4096 + k_rd[ks]);
            sacc[mt] = mfma32(a, qf[ks], sacc[mt]);
          }
      };
      if (need_mask) {
  #pragma unroll
        for (int mt = 0; mt < kMT; ++mt) {
          const uint32_t nw = ~((uint32_t)(bits >> (32 * (mt0 + mt))) >> (4 * g));   // bit set = key masked
  #pragma unroll
          for (int r = 0; r < 16; ++r) {
            // (asm: written with the builtin, the compiler turns the pair back into and + compare + select)
            int all;   // -1 if masked, else 0
            asm("v_bfe_i32 %0, %1, %2, 1" : "=v"(all) : "v"(nw), "n"(8 * (r >> 2) + (r & 3)));
            sacc[mt][r] = __builtin_bit_cast(float, (uint32_t)all & 0xFF800000u);
          }
        }
        s_product();
      } else {
  #pragma unroll
        for (int i = 0; i < kMT; ++i)
  #pragma unroll
          for (int r = 0; r < 16; ++r) sacc[i][r] = 0.f;
        s_product();
      }

      // ---- online softmax; one query per lane (shared with the partner lane ^ 32).
      // The running max is only raised when the tile's max exceeds it by more than kLazy
      // (in log2 units): probabilities then stay below 2^kLazy, well inside fp16 range, the
      // normalisation by the running sum stays exact, and the O rescale becomes rare.
      float mx = sacc[0][0];
  #pragma unroll
      for (int mt = 0; mt < kMT; ++mt)
  #pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[mt][r]);
      mx = pair_max(mx);
      const float m_new = (mx * p.c > m_run * p.c + kLazy || m_run == -INFINITY) ? mx : m_run;
      // A row that has seen no allowed key yet has m_new == -inf: subtract 0 instead, so
      // that its probabilities are exp2(-inf) = 0 and no inf - inf appears.
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_sub) * p.c);
      const float mc = m_sub * p.c;
      half8_t pf[kMT][2];   // [key sub-tile][half]: B operand of O^T = V^T . P^T
      float lsum = 0.f;
  #pragma unroll
      for (int mt = 0; mt < kMT; ++mt)
  #pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[mt][r], p.c, -mc));
          const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[mt][r + 1], p.c, -mc));
          const half2_t e2 = {(half_t)e0, (half_t)e1};
          pf[mt][r >> 3][r & 7] = e2[0];
          pf[mt][r >> 3][(r & 7) + 1] = e2[1];
          // Row sum with plain adds: v_dot2c_f32_f16 would halve the instruction count but runs
          // on the matrix pipeline and stalls behind every MFMA in flight on the SIMD.
          lsum += e0 + e1;
        }
      l_run = l_run * alpha + lsum;   // per-lane partial sum; the two halves are added at the end
      m_run = m_new;
      if (__any(alpha != 1.0f)) {
  #pragma unroll
        for (int dt = 0; dt < 2; ++dt)
  #pragma unroll
          for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
      }

      // ---- O^T += V^T . P^T
  #pragma unroll
      for (int mt = 0; mt < kMT; ++mt)
  #pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
  #pragma unroll
          for (int dt = 0; dt < 2; ++dt) {
            const lds_byte* vp = vt + (32 * (mt0 + mt) + 16 * s2) * 128;
            const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vp + v_rd[dt][0]));
            const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vp + v_rd[dt][1]));
            const half8_t a = __builtin_bit_cast(half8_t, (short8_t)__builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
            oacc[dt] = mfma32(a, pf[mt][s2], oacc[dt]);
          }
    };

    Step cur = next_step();
    if (cur.valid) issue_tile(cur.col, (lds_byte*)k_lds0, (lds_byte*)v_lds0);
    while (cur.valid) {   // single exit: an early exit between the two steps makes the compiler copy the accumulators
      Step nxt = next_step();
      step(cur, nxt, (const lds_byte*)k_lds0, (const lds_byte*)v_lds0, (lds_byte*)k_lds1, (lds_byte*)v_lds1);
      cur = nxt;
      if (nxt.valid) {
        cur = next_step();
        step(nxt, cur, (const lds_byte*)k_lds1, (const lds_byte*)v_lds1, (lds_byte*)k_lds0, (lds_byte*)v_lds0);
      }
    }
  }

  // ---- key split: the waves of the second key half hand their (max, sum, O) to the waves of
  // the first through LDS (the tile buffers are free now: the last step issued no loads), lane
  // to lane, since both hold the same queries in the same register layout.
  if (KS == 2) {
    float* xo = reinterpret_cast<float*>(half ? k_lds1 : k_lds0);   // 32 x 64 floats = one tile buffer
    float* xs = reinterpret_cast<float*>(v_lds0) + 128 * half;
    __syncthreads();
    if (mt0 == 1) {
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) xo[(16 * dt + r) * 64 + lane] = oacc[dt][r];
      xs[lane] = m_run;
      xs[64 + lane] = l_run;
    }
    __syncthreads();
    if (mt0 == 1) return;
    const float m_b = xs[lane], l_b = xs[64 + lane];
    const float m = fmaxf(m_run, m_b);
    // a side that has seen no allowed key (max still -inf) contributes nothing
    const float fa = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run - m) * p.c);
    const float fb = (m_b == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_b - m) * p.c);
    l_run = l_run * fa + l_b * fb;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] = oacc[dt][r] * fa + xo[(16 * dt + r) * 64 + lane] * fb;
  }

  // ---- normalise and store: oacc[dt][r] = O[query j32][d = 32dt + 8(r/4) + 4g + r%4]
  if (!q_valid) return;
  const float l = pair_sum(l_run);
  const float inv = (l > 0.f) ? 1.0f / l : 0.f;   // no allowed key at all: zeros
  half_t* orow = ob + (int64_t)j32 * p.os[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      half4_t o4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o4[e] = (half_t)(oacc[dt][4 * q4 + e] * inv);
      *reinterpret_cast<half4_t*>(orow + 32 * dt + 8 * q4 + 4 * g) = o4;
    }
}

// Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous range of
// (batch, head, group) so one head's K/V is read through a single L2.
__device__ __forceinline__ int xcd_contiguous_id(const AttnParams& p) {
  const int wg = blockIdx.x;
  return (wg & 7) * p.chunk + (wg >> 3);
}

// Row length usually grows (causal) or is flat along the sequence.  Workgroups are placed on
// CUs round-robin, so consecutive heads walk the sequence in opposite directions: a CU that
// receives the longest rows of one head receives the shortest rows of the next.
__device__ __forceinline__ int zigzag(int pidx, int bh, int n) {
  return ((pidx + bh) & 1) ? (pidx >> 1) : n - 1 - (pidx >> 1);   // long, short, long, ...
}

// Four distinct LDS objects (K and V, two buffers each): the compiler orders LDS reads after
// in-flight direct-to-LDS loads per object, so a read of the current buffer does not wait for
// the loads that fill the other one.
#define STOF_ATTN_LDS_TILES                                                     \
  __shared__ __attribute__((aligned(1024))) unsigned char k_lds0[kTile];        \
  __shared__ __attribute__((aligned(1024))) unsigned char k_lds1[kTile];        \
  __shared__ __attribute__((aligned(1024))) unsigned char v_lds0[kTile];        \
  __shared__ __attribute__((aligned(1024))) unsigned char v_lds1[kTile]

// Length-aware placement.  A mask with a few long rows (global rows, the bottom of a causal
// mask) otherwise leaves whole compute units with nothing but long chains: measured on B8 H12
// S1024 with two global rows, every eighth compute unit received three 16-block chains (done at
// 33 us) while most had 21 blocks in total (done at 19 us).
//
// Each XCD owns `chunk / nP` whole heads, taken in sets of about one resident round of groups
// (4 per compute unit), so that the K/V of few heads is live in the XCD's L2 at a time.  The
// groups of a set are ordered by (rank of the group inside its own head by descending row
// length, head) and dealt to the XCD's compute units, which the dispatcher fills round-robin, in
// boustrophedon order: pass 0 hands units 0..n-1 the first n groups, pass 1 hands units n-1..0
// the next n, and so on.  Sums per unit come out even and every unit starts with its longest
// chain.  The rank is computed here from the row pointers (lane l holds group l of the head; at
// most 64 groups), so no host pass over the LUT and no scratch memory is needed; being a
// permutation per head it is a bijection also when every sample has its own LUT.  The row
// pointers read for it are handed on to attn_group, which saves that a memory round trip.
template <int KIND, int ROWS>
__device__ __forceinline__ void balanced_group(const AttnParams& p, int& bh, int& pair, RowPtrs<ROWS>& pre) {
  const int lane = threadIdx.x & 63;
  const int x = blockIdx.x & 7, i = blockIdx.x >> 3;   // XCD, dispatch index inside it (i < chunk: the grid is exact)
  const int ncu = p.cus_per_xcd;
  const int hx = p.chunk / p.nP;                                        // heads of this XCD
  const int hs = min(hx, max(1, (4 * ncu + p.nP - 1) / p.nP));          // heads per set
  const int per_set = hs * p.nP;
  const int s = i / per_set;
  const int h0 = s * hs;
  const int hn = min(hs, hx - h0);                                      // heads in this set
  const int il = i - s * per_set;
  const int pass = il / ncu, pos = il - pass * ncu;
  const int plen = min(ncu, hn * p.nP - pass * ncu);
  const int j = pass * ncu + ((pass & 1) ? plen - 1 - pos : pos);       // position in the set's order
  const int rank_wanted = j / hn;
  bh = x * hx + h0 + (j - rank_wanted * hn);
  pre.valid = false;
  int rp[ROWS + 1], pp[ROWS + 1];   // LOAD / PART row pointers of group `lane`: rows ROWS*lane .. and the end
  int len = 0;
  if (KIND == kKindLut) {
    const int64_t lo = (int64_t)(bh / p.H) * p.lut_bs;
#pragma unroll
    for (int r = 0; r <= ROWS; ++r) {
      const int qr = min(ROWS * lane + r, p.nQ);   // (lanes past the last group and a missing second row read the end pointer)
      rp[r] = p.lrp[lo + qr];
      pp[r] = p.prp[lo + qr];
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) len = max(len, rp[r + 1] - rp[r]);
  } else {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int qr = ROWS * lane + r;
      const int hi = p.causal ? qr : p.nQ - 1;
      const int first_key = (KIND == kKindPred && p.band > 0) ? 64 * qr - p.band + 1 : 0;
      if (qr < p.nQ) len = max(len, hi - (first_key > 0 ? first_key / 64 : 0) + 1);
    }
  }
  // one comparable key per group: longer first, lower index first among equals
  const int key = lane < p.nP ? (len << 6) | (63 - lane) : -1;
  int rank = 0;
  for (int q = 0; q < p.nP; ++q) rank += __builtin_amdgcn_readlane(key, q) > key ? 1 : 0;
  pair = __builtin_ctzll(__ballot(lane < p.nP && rank == rank_wanted));
  if (KIND == kKindLut) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      pre.t0[r] = __builtin_amdgcn_readlane(rp[r], pair);
      pre.n[r] = __builtin_amdgcn_readlane(rp[r + 1], pair) - pre.t0[r];
      pre.p0[r] = __builtin_amdgcn_readlane(pp[r], pair);
      pre.np[r] = __builtin_amdgcn_readlane(pp[r + 1], pair) - pre.p0[r];
    }
    pre.valid = true;
  }
}

template <int KIND, int ROWS, int KS>
__global__ __launch_bounds__(128 * ROWS * KS, 4) void block_attn_fwd_kernel(const AttnParams p) {
  STOF_ATTN_LDS_TILES;
  int bh, pair;
  RowPtrs<ROWS> pre;
  pre.valid = false;
  if (p.balance) {
    balanced_group<KIND, ROWS>(p, bh, pair, pre);
  } else {
    const int vid = xcd_contiguous_id(p);
    if (vid >= p.total) return;
    bh = vid / p.nP;
    pair = zigzag(vid - bh * p.nP, bh, p.nP);
  }
  attn_group<KIND, ROWS, KS>(p, bh, pair, pre, k_lds0, k_lds1, v_lds0, v_lds1);
}

// dst[r*(cols/64)+w] bit t = pred(src[r*ld + 64w + t]).
// Vector form: a lane loads 8 elements (16 B) and forms one byte of the word; the 8 lanes of a
// word merge their bytes with three lane exchanges and the first of them stores 8 B.  A
// wavefront covers 8 consecutive words (1 KB in, 64 B out) per pass; 16-byte aligned rows only.
__global__ __launch_bounds__(256) void pack_mask_bits_vec_kernel(const half_t* __restrict__ src,
                                                                 uint64_t* __restrict__ dst,
                                                                 int64_t rows, int64_t words_per_row,
                                                                 int64_t ld, int additive) {
  const int lane = threadIdx.x & 63;
  const int sub = lane & 7;
  const int64_t nwords = rows * words_per_row;
  const int64_t stride = (int64_t)gridDim.x * 32;
  for (int64_t w0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 8; w0 < nwords; w0 += stride) {
    const int64_t w = w0 + (lane >> 3);
    uint32_t lo = 0, hi = 0;
    if (w < nwords) {
      const int64_t r = w / words_per_row;
      const int64_t cw = w - r * words_per_row;
      const half8_t x = *reinterpret_cast<const half8_t*>(src + r * ld + cw * 64 + 8 * sub);
      uint32_t byte = 0;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (float)x[e];
        byte |= (uint32_t)(additive ? (f > -5000.f) : (f > 0.f)) << e;
      }
      if (sub < 4) lo = byte << (8 * sub); else hi = byte << (8 * (sub - 4));
    }
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) {
      lo |= (uint32_t)__shfl_xor((int)lo, m, 64);
      hi |= (uint32_t)__shfl_xor((int)hi, m, 64);
    }
    if (sub == 0 && w < nwords) dst[w] = ((uint64_t)hi << 32) | lo;
  }
}

// Scalar form for rows that are not 16-byte aligned: one wavefront per 64-element word.
__global__ __launch_bounds__(256) void pack_mask_bits_kernel(const half_t* __restrict__ src,
                                                             uint64_t* __restrict__ dst,
                                                             int64_t rows, int64_t words_per_row,
                                                             int64_t ld, int additive) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nwords = rows * words_per_row;
  const int64_t stride = (int64_t)gridDim.x * 4;
  for (int64_t w = wave; w < nwords; w += stride) {
    const int64_t r = w / words_per_row;
    const int64_t cw = w - r * words_per_row;
    const float x = (float)src[r * ld + cw * 64 + lane];
    const bool keep = additive ? (x > -5000.f) : (x > 0.f);
    const uint64_t word = __ballot(keep);
    if (lane == 0) dst[w] = word;
  }
}

// Launch forms.  Two query blocks per workgroup share every K/V tile between four waves and
// halve the L2 -> LDS traffic per unit of MFMA work: the form for large grids.  (Four query
// blocks per workgroup halve it once more but measured no faster on MI355X, the kernel being
// bound by VALU/MFMA issue, not by that traffic.)  One query block per workgroup with the keys
// of each tile split over two wave pairs is the form for small grids, which are bound by the
// longest chain of key blocks: the chain runs twice as fast.
constexpr int kRowsPerGroup = 2;
enum { kFormAuto = -1, kFormTwoRows = 0, kFormKeySplit = 1 };
int g_attn_form = kFormAuto;

// Automatic choice: key split when the sequence has at least kKeySplitMinQueryBlocks query
// blocks AND the two-row grid gives a compute unit at most kKeySplitMaxGroupsPerCu workgroups.
// Four workgroups are resident per compute unit (LDS), and the key split doubles the count:
// up to two two-row groups per compute unit it still runs as a single round with every chain
// half as long (GPU time: B2 H12 S2048 causal 44 -> 34 us, B4 H12 S1024 sparse 25 -> 23 us,
// B1 H12 S512 11.1 -> 9.6 us, B1 H12 S256 7.6 -> 6.6 us), beyond that it needs a second, partly
// filled round and loses (three per compute unit: -3 % .. +15 %).  With two query blocks
// (S 128) the chains are too short either way (+-5 %).
constexpr int kKeySplitMaxGroupsPerCu = 2;
constexpr int kKeySplitMinQueryBlocks = 4;

int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  return cus;
}

int pick_form(int requested, int64_t two_row_groups, int nQ) {
  if (requested != kFormAuto) return requested;          // the caller's choice for this call
  if (g_attn_form != kFormAuto) return g_attn_form;      // the process-wide default
  return (nQ >= kKeySplitMinQueryBlocks && two_row_groups <= (int64_t)kKeySplitMaxGroupsPerCu * compute_units()) ? kFormKeySplit : kFormTwoRows;
}

// Length-aware placement needs whole heads per XCD and a compute-unit count that splits over
// the 8 XCDs.  The rank of a group costs one pass over the head's groups per workgroup: with two
// rows per workgroup it is used up to 64 groups per head (S 8192; one lane per group), with the
// key split - small grids, short kernels - up to 32 (at 64: B1 H16 S4096 +6 %).
// Measured (two rows per workgroup, zig-zag order -> length order): B8 H12 S1024 with two global
// rows 32.8 -> 26.3 us, the same mask at B4 24.9 -> 21.3, at B16 51.3 -> 48.3; causal B4 H12
// S1024 / S2048 / S4096 25.0 -> 21.0, 55.1 -> 43.3, 150 -> 141; growing-band B2 H16 S4096 46.3 ->
// 46.2, at B16 346 -> 354; dense S4096 246 -> 248; eight blocks in every row 23.8 -> 24.4; B2 H16
// S8192 band + two global rows + random blocks 178 -> 159, causal 350 -> 350.
constexpr int kBalanceMaxGroupsTwoRows = 64;
constexpr int kBalanceMaxGroupsKeySplit = 32;
void set_balance(AttnParams& p, int max_groups) {
  const int cus = compute_units();
  p.cus_per_xcd = cus / 8;
  p.balance = (p.total % 8 == 0 && p.chunk % p.nP == 0 && p.nP <= max_groups && p.nP > 1 && cus % 8 == 0 && cus >= 8) ? 1 : 0;
}

template <int KIND>
void launch_attn(AttnParams& p, int nQ, int64_t bh, int requested_form, hipStream_t stream) {
  const int64_t two_row_groups = (int64_t)((nQ + kRowsPerGroup - 1) / kRowsPerGroup) * bh;
  const int form = pick_form(requested_form, two_row_groups, nQ);
  if (form == kFormKeySplit) {
    p.nP = nQ;
    p.total = (int)(nQ * bh);
    p.chunk = (p.total + 7) / 8;
    set_balance(p, kBalanceMaxGroupsKeySplit);
    hipLaunchKernelGGL((block_attn_fwd_kernel<KIND, 1, 2>), dim3(p.chunk * 8), dim3(256), 0, stream, p);
  } else {
    p.nP = (nQ + kRowsPerGroup - 1) / kRowsPerGroup;
    p.total = (int)two_row_groups;
    p.chunk = (p.total + 7) / 8;
    set_balance(p, kBalanceMaxGroupsTwoRows);
    hipLaunchKernelGGL((block_attn_fwd_kernel<KIND, kRowsPerGroup, 1>), dim3(p.chunk * 8), dim3(128 * kRowsPerGroup), 0, stream, p);
  }
}

bool strides_ok(const int64_t s[3]) {
  return (s[0] % 8 == 0) && (s[1] % 8 == 0) && (s[2] % 8 == 0) && s[2] >= kD && s[2] < (1 << 20);
}

}  // namespace

extern "C" int stof_attn_set_launch_form(int form) {
  if (form != kFormAuto && form != kFormTwoRows && form != kFormKeySplit) return STOF_ERR_UNSUPPORTED;
  g_attn_form = form;
  return STOF_OK;
}

extern "C" int stof_block_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    const int32_t* full_row_ptr, const int32_t* full_col_idx,
    const int32_t* part_row_ptr, const int32_t* part_col_idx, const uint64_t* part_bitmask,
    const int32_t* load_row_ptr, const int32_t* load_col_idx,
    int block_m, int block_n, float softmax_scale,
    const int64_t q_strides[3], const int64_t k_strides[3],
    const int64_t v_strides[3], const int64_t out_strides[3],
    int batch_size, int seq_len, int head_num, int head_size,
    int64_t lut_batch_stride, int launch_form, void* stream) {
  if (launch_form != kFormAuto && launch_form != kFormTwoRows && launch_form != kFormKeySplit) return STOF_ERR_UNSUPPORTED;
  if (!q || !k || !v || !out || !full_row_ptr || !part_row_ptr || !load_row_ptr ||
      !q_strides || !k_strides || !v_strides || !out_strides)
    return STOF_ERR_NULL_POINTER;
  // The column lists and the bitmask may be NULL when every row range over them is empty (a
  // mask without partial blocks; a mask that allows nothing, whose output is all zeros): the
  // kernel reads them only inside non-empty row ranges.
  if (batch_size <= 0 || seq_len <= 0 || head_num <= 0 || head_size <= 0) return STOF_ERR_BAD_SHAPE;
  if (head_size != kD || block_m != kBM || block_n != kBN) return STOF_ERR_UNSUPPORTED;
  if (seq_len % kBM != 0) return STOF_ERR_BAD_SHAPE;
  const int nQ = seq_len / kBM;
  if (lut_batch_stride != 0 && lut_batch_stride < nQ + 1) return STOF_ERR_BAD_LUT;
  if (!stof_aligned16(q) || !stof_aligned16(k) || !stof_aligned16(v) || !stof_aligned16(out)) return STOF_ERR_MISALIGNED;
  if (!strides_ok(q_strides) || !strides_ok(k_strides) || !strides_ok(v_strides) || !strides_ok(out_strides))
    return STOF_ERR_MISALIGNED;
  if ((int64_t)nQ * batch_size * head_num > (int64_t)1 << 30) return STOF_ERR_BAD_SHAPE;

  AttnParams p;
  p.q = (const half_t*)q; p.k = (const half_t*)k; p.v = (const half_t*)v; p.out = (half_t*)out;
  p.prp = part_row_ptr; p.pci = part_col_idx;
  p.pbits = part_bitmask; p.lrp = load_row_ptr; p.lci = load_col_idx;
  for (int i = 0; i < 3; ++i) { p.qs[i] = q_strides[i]; p.ks[i] = k_strides[i]; p.vs[i] = v_strides[i]; p.os[i] = out_strides[i]; }
  p.lut_bs = lut_batch_stride;
  p.B = batch_size; p.S = seq_len; p.H = head_num; p.nQ = nQ;
  p.c = softmax_scale * 1.4426950408889634f;
  p.row_bits = nullptr; p.words = 0; p.causal = 0; p.band = 0;
  launch_attn<kKindLut>(p, nQ, (int64_t)batch_size * head_num, launch_form, (hipStream_t)stream);
  return stof_check_launch();
}

extern "C" int stof_rowwise_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    int kind, int is_causal, int bandwidth, const uint64_t* mask_bits,
    int batch_size, int seq_len, int head_num, int head_size, int launch_form, void* stream) {
  if (launch_form != kFormAuto && launch_form != kFormTwoRows && launch_form != kFormKeySplit) return STOF_ERR_UNSUPPORTED;
  if (!q || !k || !v || !out) return STOF_ERR_NULL_POINTER;
  if (kind != STOF_ROW_FULL && kind != STOF_ROW_SLIDING && kind != STOF_ROW_MASK) return STOF_ERR_UNSUPPORTED;
  if (kind == STOF_ROW_MASK && !mask_bits) return STOF_ERR_NULL_POINTER;
  if (batch_size <= 0 || seq_len <= 0 || head_num <= 0 || head_size <= 0) return STOF_ERR_BAD_SHAPE;
  if (head_size != kD) return STOF_ERR_UNSUPPORTED;
  if (seq_len % kBM != 0) return STOF_ERR_BAD_SHAPE;
  if (kind == STOF_ROW_SLIDING && bandwidth <= 0) return STOF_ERR_BAD_SHAPE;
  if (!stof_aligned16(q) || !stof_aligned16(k) || !stof_aligned16(v) || !stof_aligned16(out)) return STOF_ERR_MISALIGNED;
  const int nQ = seq_len / kBM;
  if ((int64_t)nQ * batch_size * head_num > (int64_t)1 << 30) return STOF_ERR_BAD_SHAPE;
  AttnParams p;
  p.q = (const half_t*)q; p.k = (const half_t*)k; p.v = (const half_t*)v; p.out = (half_t*)out;
  p.prp = nullptr; p.pci = nullptr; p.pbits = nullptr; p.lrp = nullptr; p.lci = nullptr;
  const int64_t in_s[3] = {(int64_t)head_num * seq_len * kD, (int64_t)seq_len * kD, kD};
  const int64_t out_s[3] = {(int64_t)seq_len * head_num * kD, kD, (int64_t)head_num * kD};   // [B,S,H*D]
  for (int i = 0; i < 3; ++i) { p.qs[i] = in_s[i]; p.ks[i] = in_s[i]; p.vs[i] = in_s[i]; p.os[i] = out_s[i]; }
  p.lut_bs = 0;
  p.B = batch_size; p.S = seq_len; p.H = head_num; p.nQ = nQ;
  p.c = (1.0f / sqrtf((float)head_size)) * 1.4426950408889634f;
  p.row_bits = mask_bits; p.words = seq_len / 64; p.causal = is_causal ? 1 : 0;
  p.band = kind == STOF_ROW_SLIDING ? bandwidth : 0;
  if (kind == STOF_ROW_MASK) launch_attn<kKindBits>(p, nQ, (int64_t)batch_size * head_num, launch_form, (hipStream_t)stream);
  else launch_attn<kKindPred>(p, nQ, (int64_t)batch_size * head_num, launch_form, (hipStream_t)stream);
  return stof_check_launch();
}

extern "C" int stof_pack_mask_bits(const void* src, uint64_t* dst, int64_t rows, int64_t cols, int64_t ld,
                                   int additive, void* stream) {
  if (!src || !dst) return STOF_ERR_NULL_POINTER;
  if (rows <= 0 || cols <= 0 || cols % 64 != 0 || ld < cols) return STOF_ERR_BAD_SHAPE;
  const int64_t nwords = rows * (cols / 64);
  if (ld % 8 == 0 && stof_aligned16(src)) {
    int64_t blocks = (nwords + 31) / 32;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(pack_mask_bits_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const half_t*)src, dst, rows, cols / 64, ld, additive);
  } else {
    int64_t blocks = (nwords + 3) / 4;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(pack_mask_bits_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const half_t*)src, dst, rows, cols / 64, ld, additive);
  }
  return stof_check_launch();
}
