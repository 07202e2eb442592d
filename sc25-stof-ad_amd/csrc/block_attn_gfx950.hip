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
//    (buffer_load_dwordx4 ... lds), double buffered: the loads of block t+1 are issued before
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
// Key blocks of remaining chain per issue-priority level (levels 0 .. 3: 6 and more left, 4-5, 2-3,
// under 2).  A compute unit's four workgroups arrive longest first, and among waves of equal
// priority a SIMD issues from the oldest: above the top threshold that order IS longest first.
// What the step sets is the endgame: all waves below the last threshold are equal again, the
// youngest workgroup starves and then finishes alone - about one step's worth of chain per unit
// of kPrioStep.  Measured (step 6 -> 2): B2 H16 S4096 sparse 40.4 -> 38.8 us, B4 H16 S2048 20.8 ->
// 19.0, B8 H12 S1024 21.7 -> 20.5, B16 H12 S512 14.0 -> 13.0, dense unchanged; step 1 gives back 1-5 %.
constexpr int kPrioStep = 2;

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
  // precomputed walk (see attn_plan_kernel): one block of plan_stride 8-byte words per (LUT sample, group slot)
  const uint64_t* plan; int plan_stride;
};

enum { kKindLut = 0, kKindPred = 1, kKindBits = 2 };

typedef unsigned short ushort8_t __attribute__((ext_vector_type(8)));

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
template <int KIND, int ROWS, int KS, bool PIPE, bool BF, bool PLAN = false>
__device__ __forceinline__ void attn_group(const AttnParams& p, const int bh, const int pair_or_slot, const RowPtrs<ROWS>& pre,
                                           unsigned char* k_lds0, unsigned char* k_lds1,
                                           unsigned char* v_lds0, unsigned char* v_lds1,
                                           unsigned char* k_lds2 = nullptr, unsigned char* v_lds2 = nullptr) {
  static_assert(KS == 1 || ROWS == 1, "the key split serves a single query block");
  static_assert(!PIPE || KS == 1, "the software-pipelined loop keeps all 64 keys of a tile in one wave");
  static_assert(!PLAN || (KIND == kKindLut && !PIPE), "a precomputed walk exists for LUT-driven launches of the plain loop");
  // PLAN: the group's walk was laid out ahead of time.  Lane l takes word l of the group's plan
  // block; this one load, issued first of all, replaces the row pointers, the column lists and the
  // merge of the rows - two dependent round trips through memory and some hundred scalar
  // instructions between the start of the workgroup and its first K/V tile.
  int pair = pair_or_slot;
  uint32_t plan_lo = 0, plan_hi = 0;     // the current window of 64 plan words, one per lane
  uint64_t plan_sw[4] = {0, 0, 0, 0};    // words 0-3 of the block in scalar registers (a block has at least 8 words)
  const uint64_t* plan_blk = nullptr;
  if constexpr (PLAN) {
    const int sample = p.lut_bs ? bh / p.H : 0;
    plan_blk = p.plan + ((int64_t)sample * p.nP + pair_or_slot) * p.plan_stride;
    const int l = threadIdx.x & 63;
    const uint64_t w = l < p.plan_stride ? plan_blk[l] : 0ull;
    plan_lo = (uint32_t)w; plan_hi = (uint32_t)(w >> 32);
    // the header and the first two steps also through the scalar cache: a wave-uniform address, and the
    // answer does not queue behind the vector-memory traffic of the sixteen waves that start together
#pragma unroll
    for (int i = 0; i < 4; ++i) plan_sw[i] = plan_blk[i];
  }
  constexpr int kDma = 4 / (ROWS * KS);   // direct-to-LDS instructions per wave and operand tile (8 per tile)
  constexpr int kMT = 2 / KS;             // 32-key sub-tiles of a key block handled by one wave

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int j32 = lane & 31;
  const int g = lane >> 5;
  const int rsel = KS == 1 ? wave >> 1 : 0;   // which of the group's query blocks this wave serves
  const int half = wave & 1;                  // which 32 queries of that block
  const int mt0 = KS == 1 ? 0 : wave >> 1;    // first 32-key sub-tile of this wave
  // Accumulator start values of partial tiles: entry n (a nibble of the inverted mask word: bit e
  // set = key e of four masked) holds four floats, -inf where masked and 0 where allowed.
  __shared__ __attribute__((aligned(256))) float mask_tab[64];
  if (wave == 0) mask_tab[lane] = ((lane >> 2) >> (lane & 3)) & 1 ? -INFINITY : 0.f;

  int plan_n = 0, plan_p0 = 0, plan_i = 0;   // PLAN: steps of the group, first PART slot of this wave's row, next step
  if constexpr (PLAN) {
    const uint32_t h0 = (uint32_t)plan_sw[0];
    pair = h0 & 0xffff;
    plan_n = h0 >> 16;
    plan_p0 = rsel == 0 ? (int)(uint32_t)plan_sw[1] : (int)(uint32_t)(plan_sw[1] >> 32);
  }
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
      if (PLAN) {
        row[r].n = plan_n;
      } else if (KIND == kKindLut) {
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
    if (PLAN) return;
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
  float mc_run = 0.f;      // running max * c, what the exponent subtracts
  bool warm = false;       // every lane of the wave has a finite running max
  constexpr float kSumLimit = 16384.f;   // 32 probabilities of at most 2^kLazy sum to 2^13

  // K and V of this (batch, head) as buffer resources: a tile load is then the resource (scalar
  // registers, set up once), the tile's byte offset (one scalar multiply) and the lane's 32-bit
  // offset inside a tile - no 64-bit address arithmetic per tile.  The byte span of a head is below
  // 2^31 (checked by the host), and the resource's extent is that span, so an offset beyond the
  // tensor would read zeros instead of faulting.
  const uint32_t k_tile_bytes = (uint32_t)(kBN * 2 * p.ks[2]), v_tile_bytes = (uint32_t)(kBN * 2 * p.vs[2]);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(kb), 0, (int)(((int64_t)(p.S - 1) * p.ks[2] + kD) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(vb), 0, (int)(((int64_t)(p.S - 1) * p.vs[2] + kD) * 2), 0x00020000);
  auto issue_tile = [&](int col, lds_byte* kdst, lds_byte* vdst) {
    const uint32_t kt = (uint32_t)col * k_tile_bytes, vt = (uint32_t)col * v_tile_bytes;
    lds_byte* kd = kdst + (kDma * wave) * 1024;
    lds_byte* vd = vdst + (kDma * wave) * 1024;
#pragma unroll
    for (int i = 0; i < kDma; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (__attribute__((address_space(3))) void*)(kd + i * 1024), 16, k_src[i], kt, 0, 0);
#pragma unroll
    for (int i = 0; i < kDma; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (__attribute__((address_space(3))) void*)(vd + i * 1024), 16, v_src[i], vt, 0, 0);
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
  if (!PLAN) consume_window(0);
  uint32_t plan_nlo = 0, plan_nhi = 0;   // PLAN: the window after the current one, requested 16 steps before it is needed
  auto next_step = [&]() -> Step {
    Step s; s.col = 0; s.mine = 0; s.slot = -1; s.valid = false;
    if constexpr (PLAN) {
      // word 2 + i of the block is step i: key block (16 bits), listed by row 0 / row 1, partial in
      // row 0 / row 1 (bits 16-19), and in the upper half the PART slots relative to the rows' first
      if (plan_i >= plan_n) return s;
      const int word = plan_i + 2;
      if ((word & 63) == 0) { plan_lo = plan_nlo; plan_hi = plan_nhi; }
      uint32_t lo, hi;
      if (word < 4) {   // the first two steps: from the scalar copy, without waiting for the window
        const uint64_t w = word == 2 ? plan_sw[2] : plan_sw[3];
        lo = (uint32_t)w; hi = (uint32_t)(w >> 32);
      } else {
        lo = __builtin_amdgcn_readlane(plan_lo, word & 63);
        hi = __builtin_amdgcn_readlane(plan_hi, word & 63);
      }
      if ((word & 63) == 48 && (word | 63) + 1 < plan_n + 2) {
        const int at = (word | 63) + 1 + lane;
        const uint64_t w = at < p.plan_stride ? plan_blk[at] : 0ull;
        plan_nlo = (uint32_t)w; plan_nhi = (uint32_t)(w >> 32);
      }
      ++plan_i;
      s.valid = true;
      s.col = lo & 0xffff;
      s.mine = (lo >> (16 + rsel)) & 1;
      if (s.mine && ((lo >> (18 + rsel)) & 1)) s.slot = plan_p0 + ((hi >> (16 * rsel)) & 0xffff);
      return s;
    }
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
    // ---- software-pipelined main loop, in units of HALF a tile (32 keys x this wave's 32 queries).
    // For unit u the wave has three pieces of work: A(u) its scores S = K Q^T (4 MFMA), B(u) its
    // probabilities exp2(S c - m c) with their row sum (vector ALU only) and C(u) its share of
    // O += V^T P^T (4 MFMA).  A half-step runs A(u+1), B(u) and C(u-1) together: they are
    // independent of one another, so inside ONE wave every MFMA is followed by vector-ALU work
    // that does not wait for it, and the matrix pipeline and the vector ALU run side by side.
    // (Across waves they overlap badly: an MFMA that waits for the pipeline holds the SIMD's
    // issue slot.)  Per tile i, between two barriers, the wave runs two half-steps,
    //     A(i, keys 32-63) | B(i, keys 0-31)  | C(i-1, keys 32-63)
    //     A(i+1, keys 0-31) | B(i, keys 32-63) | C(i, keys 0-31)
    // so one unit of scores (16 registers) and one unit of probabilities (8) cross an iteration.
    //
    // There is ONE code path for every unit (two paths that both update the accumulators cost
    // some 90 registers at their merge points).  What differs is decided by small side blocks:
    //  * a unit of a tile the wave's row does not list, or of a slot before the first / after
    //    the last tile, is computed like any other but subtracts +inf in the exponent, so its
    //    probabilities are exactly zero (the tile buffers are zero-filled once at the start, so
    //    every operand is finite);
    //  * a masked unit has -inf added to the scores of its masked elements, in place, before its
    //    softmax;
    //  * the running max: normally it is taken as it stands and the unit only verifies, from the
    //    row sum it needs anyway, that no probability left the fp16 range (the max would have to
    //    rise by more than 2^14 inside one unit).  While a lane has not seen a key yet the unit is
    //    preceded by the exact update (max search, lazy raise, rescale of O, of the sum and of
    //    the previous unit's probabilities, which go into O during this half-step).  A failed
    //    verification raises a flag, and once the walk is over a workgroup with a raised flag
    //    runs the whole walk a second time with the exact update before every unit.
    //
    // LDS: rings of three K and three V tiles.  Iteration i reads K(i), K(i+1), V(i-1), V(i) and
    // issues the loads of K(i+2) and V(i+1) into the buffers iteration i-1 read last.
    enum { kValid = 1, kMine = 2, kMask = 4 };   // tile flags: listed by the walk, used by this wave's row, needs its element mask
    struct Tile { int col, slot, f; };
    auto dma_k = [&](int col, lds_byte* kdst) {
      const uint32_t kt = (uint32_t)col * k_tile_bytes;
      lds_byte* kd = kdst + (kDma * wave) * 1024;
#pragma unroll
      for (int i = 0; i < kDma; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (__attribute__((address_space(3))) void*)(kd + i * 1024), 16, k_src[i], kt, 0, 0);
    };
    auto dma_v = [&](int col, lds_byte* vdst) {
      const uint32_t vt = (uint32_t)col * v_tile_bytes;
      lds_byte* vd = vdst + (kDma * wave) * 1024;
#pragma unroll
      for (int i = 0; i < kDma; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (__attribute__((address_space(3))) void*)(vd + i * 1024), 16, v_src[i], vt, 0, 0);
    };
    // element-mask word of this lane's query for a tile (requested when the tile enters the queue)
    auto request_bits = [&](const Tile& t) -> uint64_t {
      uint64_t bits = ~0ull;
      if (KIND == kKindLut) {
        if (t.slot >= 0) bits = p.pbits[(int64_t)t.slot * kBM + 32 * half + j32];
      } else if (KIND == kKindBits) {
        if (t.f & kMine) bits = p.row_bits[(qrow0 + j32) * p.words + t.col];
      }
      return bits;
    };
    // whether the tile needs its element mask (wave-uniform); the index predicates of the
    // row-wise front-ends are folded into the bit row; a tile that allows nothing is dropped
    auto settle_mask = [&](Tile& t, uint64_t& bits) {
      if (KIND == kKindLut) return;                  // decided by the walk: a PART slot
      if (!(t.f & kMine)) return;
      const int qmin = (int)qrow0, qmax = qmin + 31, kmin = t.col * kBN, kmax = kmin + kBN - 1;
      const bool range_full = (!p.causal || kmax <= qmin) && (!(KIND == kKindPred && p.band > 0) || kmin > qmax - p.band);
      bool mask;
      if (KIND == kKindBits) {
        if (!__any(bits != 0ull)) { t.f &= ~kMine; return; }
        mask = !range_full || __any(bits != ~0ull);
      } else {
        mask = !range_full;
      }
      if (mask) {
        t.f |= kMask;
        const int qg = qmin + j32;
        if (p.causal) { const int nk = qg - kmin + 1; bits &= nk >= 64 ? ~0ull : (nk <= 0 ? 0ull : ((1ull << nk) - 1)); }
        if (KIND == kKindPred && p.band > 0) {
          const int first = qg - p.band + 1 - kmin;
          bits &= first <= 0 ? ~0ull : (first >= 64 ? 0ull : ~((1ull << first) - 1));
        }
      }
    };
    // Element mask of a unit, applied to its finished scores in place: -inf where the key is not
    // allowed (added as a 0 / -inf bias: sign-extended one-bit field of the inverted mask word,
    // AND with the bit pattern of -inf, add).
    auto apply_mask = [&](floatx16& sc, uint32_t unit_bits) {
      const uint32_t nw = ~(unit_bits >> (4 * g));   // bit set = key masked
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        int all;   // -1 if masked, else 0
        asm("v_bfe_i32 %0, %1, %2, 1" : "=v"(all) : "v"(nw), "n"(8 * (r >> 2) + (r & 3)));
        sc[r] += __builtin_bit_cast(float, (uint32_t)all & 0xFF800000u);
      }
    };
    // vh: the unit's half of a V tile buffer (key rows 32 mt .. 32 mt + 31)
    auto v_frag = [&](const lds_byte* vh, int s2, int dt) -> half8_t {
      const lds_byte* vp = vh + 16 * s2 * 128;
      const short4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vp + v_rd[dt][0]));
      const short4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vp + v_rd[dt][1]));
      return __builtin_bit_cast(half8_t, (short8_t)__builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    // Exact update of the running max ahead of a unit's softmax: s = the unit's scores, p_prev =
    // the previous unit's probabilities (they enter O during this half-step, so they are brought
    // to the new max along with O and the running sum).
    auto exact_update = [&](const floatx16& s, half8_t (&p_prev)[2]) {
      float mx = s[0];
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
      mx = pair_max(mx);
      const float m_new = (mx * p.c > m_run * p.c + kLazy || m_run == -INFINITY) ? mx : m_run;
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_sub) * p.c);
      mc_run = m_sub * p.c;
      m_run = m_new;
      l_run *= alpha;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          // (bf16 -> fp32 as a shift of the whole vector's bit patterns: casting single elements
          // of the half-typed container to __bf16 is miscompiled by this toolchain)
          const ushort8_t bits16 = __builtin_bit_cast(ushort8_t, p_prev[s2]);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            if constexpr (BF) p_prev[s2][e] = to_elem<BF>(__builtin_bit_cast(float, (uint32_t)bits16[e] << 16) * alpha);
            else p_prev[s2][e] *= (half_t)alpha;
          }
        }
      }
      warm = !__any(m_run == -INFINITY);
    };

    // The walk as a table.  Finding the next key block in the bit sets costs some twenty scalar
    // instructions per tile, which a wave issues one at a time between its vector work; with few
    // waves per SIMD nothing hides them.  Per window of 64 key blocks the walk is therefore laid
    // out once: the k-th block of the union goes to lane k of `table` (column inside the window,
    // whether this wave's row lists it, whether it is partial there, and its rank in the row's
    // PART list), by one forward lane permutation; a step is then one v_readlane.
    int table = 0, tab_n = 0, tab_i = 0;
    auto build_table = [&]() {
      const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
      const int rank = __builtin_popcountll(set_union & below);
      tab_n = __builtin_popcountll(set_union);
      tab_i = 0;
      const bool in_u = (set_union >> lane) & 1;
      const int dst = in_u ? rank : tab_n + (lane - rank);          // a permutation of the 64 lanes
      const int info = lane | ((int)((set_mine >> lane) & 1) << 6) | ((int)((set_part >> lane) & 1) << 7) |
                       (__builtin_popcountll(set_part & below) << 8);
      table = __builtin_amdgcn_ds_permute(dst << 2, info);
      set_union = 0;   // the window is handed out through the table from here on
    };
    build_table();   // window 0 (consumed above)
    auto next_tile = [&]() -> Tile {
      Tile t; t.col = 0; t.slot = -1; t.f = 0;
      while (tab_i >= tab_n) {
        if (++win >= n_win) return t;
        fetch_window();
        consume_window(win);
        build_table();
      }
      const int info = __builtin_amdgcn_readlane(table, tab_i++);
      t.col = 64 * win + (info & 63);
      t.f = kValid | ((info >> 5) & kMine);                        // bit 6 of the entry
      if (KIND == kKindLut && (info & 0xC0) == 0xC0) { t.slot = part_base + (info >> 8); t.f |= kMask; }
      return t;
    };

    Tile t0, t1, t2, t3;   // tiles i-1, i, i+1, i+2 of the walk
    uint64_t bits1 = ~0ull, bits2 = ~0ull;   // mask words of tiles t1 and t2
    int prio_in = 1;
    floatx16 sU, sN;       // scores: of the unit whose softmax is next, of the unit after it
    half8_t pU[2], pN[2];  // probabilities: of the unit whose PV product is next, of the unit after it
    bool safe = false;       // second pass: exact path only
    bool overflow = false;   // a fast unit failed its verification
    const int chain_len = steps_left;

    // One half-step: 8 slices, slice c = MFMA c (even: A, odd: C), the LDS fragment of a later
    // MFMA and the softmax of one pair of scores (2 fma, 2 exp2, 1 convert, 1 packed add: about
    // the issue time of the MFMA).  The slices are fenced so that the compiler keeps this order;
    // inside a slice it is free.  Returns the unit's row sum.  frag[] holds the operands of this
    // half-step's MFMAs (the first kAhead requested by the caller); fetch_next requests operands
    // of the half-step that follows, so that its first MFMAs do not wait for LDS.
    // sub: the exponent's subtrahend, mc_run or +inf (a unit that is not this wave's).
    constexpr int kAhead = 2;
    auto half_step = [&](auto&& fetch_this, auto&& fetch_next, half8_t (&frag)[8], half8_t (&frag_next)[8], bool has_next,
                         const floatx16& s_in, floatx16& s_out, const half8_t (&p_in)[2], half8_t (&p_out)[2],
                         float sub) -> float {
#pragma unroll
      for (int r = 0; r < 16; ++r) s_out[r] = 0.f;
      half2_t part[4];
      float fsum = 0.f;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        __builtin_amdgcn_sched_barrier(0);
        const int j = c >> 1;
        if (c & 1) oacc[j & 1] = mfma32<BF>(frag[c], p_in[j >> 1], oacc[j & 1]);
        else s_out = mfma32<BF>(frag[c], qf[j], s_out);
        if (c + kAhead < 8) frag[c + kAhead] = fetch_this(c + kAhead);
        else if (has_next) frag_next[c + kAhead - 8] = fetch_next(c + kAhead - 8);
        const int r = 2 * c;
        const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_in[r], p.c, -sub));
        const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_in[r + 1], p.c, -sub));
        const half2_t e2 = {to_elem<BF>(e0), to_elem<BF>(e1)};
        p_out[r >> 3][r & 7] = e2[0];
        p_out[r >> 3][(r & 7) + 1] = e2[1];
        if constexpr (BF) fsum = c == 0 ? e0 + e1 : fsum + (e0 + e1);   // (bf16 keeps 8 bits: sum in fp32)
        else part[c & 3] = c < 4 ? e2 : part[c & 3] + e2;
      }
      __builtin_amdgcn_sched_barrier(0);
      // (Pin the probabilities here: being pure arithmetic that is only read by the next half-step,
      // they would otherwise be sunk out of the slices, past the side blocks in between.)
      asm volatile("" : "+v"(p_out[0]), "+v"(p_out[1]));
      if constexpr (BF) return fsum;
      const half2_t tot = (part[0] + part[1]) + (part[2] + part[3]);
      return (float)tot[0] + (float)tot[1];
    };

    // One iteration.  k_cur / k_nxt / v_prv / v_cur: the ring buffers of K(i), K(i+1), V(i-1), V(i);
    // k_fill / v_fill: where K(i+2) and V(i+1) go.
    auto iteration = [&](const lds_byte* k_cur, const lds_byte* k_nxt, const lds_byte* v_prv, const lds_byte* v_cur,
                         lds_byte* k_fill, lds_byte* v_fill) {
      if (--prio_in == 0) {   // issue priority by remaining chain length, looked at once per kPrioStep tiles
        prio_in = kPrioStep;
        steps_left -= kPrioStep;
        if (steps_left >= 3 * kPrioStep) __builtin_amdgcn_s_setprio(3);
        else if (steps_left >= 2 * kPrioStep) __builtin_amdgcn_s_setprio(2);
        else if (steps_left >= kPrioStep) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): K(i+1), V(i) and the mask word of tile i+1 have landed
      __syncthreads();
      if (t3.f & kValid) dma_k(t3.col, k_fill);
      if (t2.f & kValid) dma_v(t2.col, v_fill);
      const uint64_t bits3 = request_bits(t3);
      settle_mask(t2, bits2);
      const lds_byte* ka = k_cur + 4096;   // A(i, keys 32-63)
      const lds_byte* kb2 = k_nxt;         // A(i+1, keys 0-31)
      const lds_byte* va = v_prv + 4096;   // C(i-1, keys 32-63)
      const lds_byte* vb2 = v_cur;         // C(i, keys 0-31)
      half8_t f1[8], f2[8];
      auto fetch1 = [&](int m) -> half8_t {
        if (m & 1) return v_frag(va, (m >> 1) >> 1, (m >> 1) & 1);
        return *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(ka + k_rd[m >> 1]);
      };
      auto fetch2 = [&](int m) -> half8_t {
        if (m & 1) return v_frag(vb2, (m >> 1) >> 1, (m >> 1) & 1);
        return *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(kb2 + k_rd[m >> 1]);
      };
#pragma unroll
      for (int m = 0; m < kAhead; ++m) f1[m] = fetch1(m);
      const bool mine1 = (t1.f & kMine) != 0;
      const bool exact = mine1 && (safe || !warm);
      const bool mask1 = (t1.f & kMask) != 0;
      // ---- half-step 1: A(i, keys 32-63) -> sN | B(i, keys 0-31): sU -> pN | C(i-1, keys 32-63): pU
      if (mask1) apply_mask(sU, (uint32_t)bits1);
      if (exact) exact_update(sU, pU);
      const float sum1 = half_step(fetch1, fetch2, f1, f2, true, sU, sN, pU, pN, mine1 ? mc_run : INFINITY);
      l_run += sum1;
      // ---- half-step 2: A(i+1, keys 0-31) -> sU | B(i, keys 32-63): sN -> pU | C(i, keys 0-31): pN
      if (mask1) apply_mask(sN, (uint32_t)(bits1 >> 32));
      if (mine1 && (safe || !warm)) exact_update(sN, pN);
      const float sum2 = half_step(fetch2, fetch2, f2, f1, false, sN, sU, pN, pU, mine1 ? mc_run : INFINITY);
      l_run += sum2;
      overflow |= __any(!(sum1 < kSumLimit) || !(sum2 < kSumLimit));
      t0 = t1; t1 = t2; t2 = t3;
      bits1 = bits2; bits2 = bits3;
      t3 = next_tile();
    };

    // The tile buffers start as zeros: a slot before the first tile is then read as finite numbers.
    {
      const floatx4 z = {0.f, 0.f, 0.f, 0.f};
      unsigned char* bufs[6] = {k_lds0, k_lds1, k_lds2, v_lds0, v_lds1, v_lds2};
#pragma unroll
      for (int bI = 0; bI < 6; ++bI)
#pragma unroll
        for (int i = 0; i < kTile / (256 * 16); ++i) *reinterpret_cast<floatx4*>(bufs[bI] + (i * 256 + threadIdx.x) * 16) = z;
    }

    for (;;) {
      t0.col = t1.col = t2.col = 0; t0.slot = t1.slot = t2.slot = -1; t0.f = t1.f = t2.f = 0;
      t3 = next_tile();
      bits1 = bits2 = ~0ull;
      prio_in = 1;                           // (the first iteration sets the priority)
      steps_left = chain_len + kPrioStep;
#pragma unroll
      for (int r = 0; r < 16; ++r) { sU[r] = 0.f; sN[r] = 0.f; }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int e = 0; e < 8; ++e) { pU[s2][e] = (half_t)0.f; pN[s2][e] = (half_t)0.f; }
      while ((t0.f | t1.f | t2.f | t3.f) & kValid) {   // single exit; tile i uses ring slot (i + 2) mod 3
        iteration((const lds_byte*)k_lds0, (const lds_byte*)k_lds1, (const lds_byte*)v_lds2, (const lds_byte*)v_lds0, (lds_byte*)k_lds2, (lds_byte*)v_lds1);
        iteration((const lds_byte*)k_lds1, (const lds_byte*)k_lds2, (const lds_byte*)v_lds0, (const lds_byte*)v_lds1, (lds_byte*)k_lds0, (lds_byte*)v_lds2);
        iteration((const lds_byte*)k_lds2, (const lds_byte*)k_lds0, (const lds_byte*)v_lds1, (const lds_byte*)v_lds2, (lds_byte*)k_lds1, (lds_byte*)v_lds0);
      }
      if (safe) break;
      // Did a fast unit of any of the four waves fail its verification?  (They share the tile
      // loads and the barriers, so the workgroup repeats the walk as a whole.)
      int* flag = reinterpret_cast<int*>(k_lds0);
      __syncthreads();                              // every wave is out of the loop: the tile buffers are free
      if (threadIdx.x == 0) *flag = 0;
      __syncthreads();
      if (overflow && lane == 0) *flag = 1;
      __syncthreads();
      const int again = __builtin_amdgcn_readfirstlane(*reinterpret_cast<volatile int*>(flag));
      __syncthreads();
      if (!again) break;
      // second pass from the start of the walk, exact path only
      safe = true;
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
      m_run = -INFINITY; l_run = 0.f; mc_run = 0.f; warm = false;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) { row[r].ptr = 0; row[r].pptr = 0; }
      win = 0;
      fetch_window();
      consume_window(0);
      build_table();
    }
  } else {
    float raise_at = -INFINITY;   // (running max) * c + kLazy: a tile max above it raises the running max
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
      // the key is allowed, -inf where it is not (-inf + finite = -inf), instead of test + compare
      // + select after the product.  The start values come four at a time from a 16-entry table
      // in LDS, indexed by a nibble of the inverted mask word (two vector instructions and one
      // 16-byte LDS read per four keys; forming them in registers - sign-extended one-bit field,
      // AND with the pattern of -inf - took eight: a mask of partial tiles only 41.8 -> 39.9 us,
      // B4 H16 S2048 causal window + global 24.5 -> 23.9, same bits).  The two cases run their own
      // copy of the product so that the unmasked one keeps the constant-zero accumulator input.
      floatx16 sacc[kMT];
      auto s_product = [&]() {
  #pragma unroll
        for (int ks = 0; ks < 4; ++ks)
  #pragma unroll
          for (int mt = 0; mt < kMT; ++mt) {
            const half8_t a = *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(kt + (mt0 + mt) * 4096 + k_rd[ks]);
            sacc[mt] = mfma32<BF>(a, qf[ks], sacc[mt]);
          }
      };
      if (need_mask) {
  #pragma unroll
        for (int mt = 0; mt < kMT; ++mt) {
          const uint32_t nw = ~((uint32_t)(bits >> (32 * (mt0 + mt))) >> (4 * g));   // bit set = key masked
  #pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            // four consecutive keys = one nibble of the mask word = one 16-byte entry of the table
            const uint32_t off = (q4 == 0 ? (nw << 4) : (nw >> (8 * q4 - 4))) & 0xF0u;
            const floatx4 t = *reinterpret_cast<const __attribute__((address_space(3))) floatx4*>((const lds_byte*)mask_tab + off);
  #pragma unroll
            for (int e = 0; e < 4; ++e) sacc[mt][4 * q4 + e] = t[e];
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
      auto raise_max = [&]() {
        float mx = sacc[0][0];
#pragma unroll
        for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[mt][r]);
        mx = pair_max(mx);
        // Nothing to do unless some lane's tile max exceeds its threshold (running max + kLazy, in
        // log2 units; -inf for a row that has seen no key, so its first finite score gets here):
        // one multiply and one compare on the common path.
        if (!__any(mx * p.c > raise_at)) return;
        const float m_new = (mx * p.c > raise_at) ? mx : m_run;
        // A row that has seen no allowed key yet has m_new == -inf: subtract 0 instead, so
        // that its probabilities are exp2(-inf) = 0 and no inf - inf appears.
        const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_sub) * p.c);
        mc_run = m_sub * p.c;
        raise_at = m_new * p.c + kLazy;
        l_run *= alpha;   // per-lane partial sum; the two halves are added at the end
        m_run = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
          for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
        }
      };
      half8_t pf[kMT][2];   // [key sub-tile][half]: B operand of O^T = V^T . P^T
      auto probabilities = [&]() -> float {
        half2_t part[4];   // four interleaved partial sums of at most 8 values each
        float fsum = 0.f;
#pragma unroll
        for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[mt][r], p.c, -mc_run));
            const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[mt][r + 1], p.c, -mc_run));
            const half2_t e2 = {to_elem<BF>(e0), to_elem<BF>(e1)};
            pf[mt][r >> 3][r & 7] = e2[0];
            pf[mt][r >> 3][(r & 7) + 1] = e2[1];
            if constexpr (BF) { fsum += e0 + e1; continue; }   // (bf16 keeps 8 bits: sum in fp32)
            // Row sum with packed fp16 adds on the values the second product uses, folded to fp32
            // once per tile (v_dot2c_f32_f16 would do it in one instruction per pair but runs on
            // the matrix pipeline and stalls behind every MFMA in flight on the SIMD).
            const int i = (r >> 1) & 3;
            part[i] = (mt == 0 && r < 8) ? e2 : part[i] + e2;
          }
        if constexpr (BF) return fsum;
        const half2_t tot = (part[0] + part[1]) + (part[2] + part[3]);
        return (float)tot[0] + (float)tot[1];
      };
      raise_max();
      l_run += probabilities();

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
            oacc[dt] = mfma32<BF>(a, pf[mt][s2], oacc[dt]);
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

  // ---- normalise and store: oacc[dt][r] = O[query j32][d = 32dt + 8(r/4) + 4g + r%4].  In that
  // layout a store instruction would write 16 B into each of 32 rows (32 partial cache lines),
  // so the wave's 32 x 64 block goes through 4 KB of LDS of its own (the tile buffers are free
  // once every wave has left the walk; 16-byte chunks XOR-ed by the row so that the row-wise
  // reads are conflict-free) and leaves as 4 stores of 8 full 128-byte rows each.
  if (KS == 1) __syncthreads();   // (the key split has passed its own barriers above)
  if (!q_valid) return;
  const float l = pair_sum(l_run);
  const float inv = (l > 0.f) ? 1.0f / l : 0.f;   // no allowed key at all: zeros
  lds_byte* stage = (lds_byte*)(KS == 2 ? v_lds1 : (wave < 2 ? k_lds0 : k_lds1)) + (wave & 1) * 4096;   // (key split: waves 0 and 1 are left)
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      half4_t o4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o4[e] = to_elem<BF>(oacc[dt][4 * q4 + e] * inv);
      *reinterpret_cast<__attribute__((address_space(3))) half4_t*>(stage + j32 * 128 + (((4 * dt + q4) ^ (j32 & 7)) << 4) + 8 * g) = o4;
    }
  const __amdgpu_buffer_rsrc_t o_rsrc = stof_wave_rsrc(ob);   // this wave's 32 output rows (their span is below 2^31 bytes: see strides_ok)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = 8 * i + (lane >> 3), c = lane & 7;
    const half8_t o = *reinterpret_cast<const __attribute__((address_space(3))) half8_t*>(stage + t * 128 + ((c ^ (t & 7)) << 4));
    // Written THROUGH the XCD's cache (device scope): the rows leave for memory while the kernel
    // still runs.  As plain cached stores they sit in L2 until the end-of-kernel write-back, which
    // the next launch waits for: B2 H16 S4096 sparse 40.3 -> 39.4 us per launch, B8 H12 S1024
    // 22.5 -> 21.0, B16 H12 S512 15.6 -> 14.0; inside an encoder layer the following GEMM reads the
    // rows at the same speed (a non-temporal store measured the same alone but slowed that GEMM).
    stof_store16_through(o_rsrc, (uint32_t)t * (uint32_t)(p.os[2] * 2) + 16 * c, o);
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

// The placement arithmetic of balanced_group alone: which (batch, head) and which position of
// the head's length order this workgroup takes.  With a precomputed walk the groups of a LUT
// are stored in that order already, so nothing has to be read or ranked here.
__device__ __forceinline__ void balanced_slot(const AttnParams& p, int& bh, int& slot) {
  const int x = blockIdx.x & 7, i = blockIdx.x >> 3;
  const int ncu = p.cus_per_xcd;
  const int hx = p.chunk / p.nP;
  const int hs = min(hx, max(1, (4 * ncu + p.nP - 1) / p.nP));
  const int per_set = hs * p.nP;
  const int s = i / per_set;
  const int h0 = s * hs;
  const int hn = min(hs, hx - h0);
  const int il = i - s * per_set;
  const int pass = il / ncu, pos = il - pass * ncu;
  const int plen = min(ncu, hn * p.nP - pass * ncu);
  const int j = pass * ncu + ((pass & 1) ? plen - 1 - pos : pos);
  slot = j / hn;
  bh = x * hx + h0 + (j - slot * hn);
}

template <int KIND, int ROWS, int KS, bool BF, bool PLAN>
__global__ __launch_bounds__(128 * ROWS * KS, 4) void block_attn_fwd_kernel(const AttnParams p) {
  STOF_ATTN_LDS_TILES;
  int bh, pair;
  RowPtrs<ROWS> pre;
  pre.valid = false;
  if (p.balance) {
    if constexpr (PLAN) balanced_slot(p, bh, pair);
    else balanced_group<KIND, ROWS>(p, bh, pair, pre);
  } else {
    const int vid = xcd_contiguous_id(p);
    if (vid >= p.total) return;
    bh = vid / p.nP;
    pair = zigzag(vid - bh * p.nP, bh, p.nP);   // (PLAN: a position of the length order - any bijection serves)
  }
  attn_group<KIND, ROWS, KS, false, BF, PLAN>(p, bh, pair, pre, k_lds0, k_lds1, v_lds0, v_lds1);
}

// ---- the walk of every group of a LUT, laid out once per LUT -----------------------------------
// One block of `stride` 8-byte words per (LUT sample, slot), slot = the group's place when the
// sample's groups are ordered by descending number of steps (ties: lower group first; more than
// 64 groups per sample: slot = group).  Word 0: group index (bits 0-15), number of steps (16-31).
// Word 1: first PART slot of the group's row 0 (low half) and row 1 (high half).  Word 2 + i, step
// i of the merged ascending walk over the rows' LOAD lists: key block (bits 0-15), listed by row
// 0 / row 1 (bits 16, 17), partial in row 0 / row 1 (bits 18, 19), PART slot relative to the
// row's first, row 0 in bits 32-47 and row 1 in bits 48-63.
constexpr int kPlanMaxKeyBlocks = 1024;   // seq_len <= 65536
__host__ __device__ inline int plan_stride_words(int nK) { return (nK + 2 + 7) & ~7; }

template <int ROWS>
__global__ __launch_bounds__(64) void attn_plan_kernel(const int32_t* __restrict__ lrp, const int32_t* __restrict__ lci,
                                                       const int32_t* __restrict__ prp, const int32_t* __restrict__ pci,
                                                       int64_t lut_bs, int nQ, int nK, int nP, int stride,
                                                       uint64_t* __restrict__ plan) {
  __shared__ unsigned char listed[ROWS][kPlanMaxKeyBlocks];
  __shared__ unsigned char partial[ROWS][kPlanMaxKeyBlocks];
  __shared__ unsigned short pslot[ROWS][kPlanMaxKeyBlocks];
  const int lane = threadIdx.x;
  const int sample = blockIdx.x / nP, g = blockIdx.x - sample * nP;
  const int64_t lo = (int64_t)sample * lut_bs;
  auto clampn = [&](int n) { return n < 0 ? 0 : (n > nK ? nK : n); };

  // the slot: rank of this group among the sample's groups by merged walk length
  int slot = g;
  if (nP <= 64) {
    int len = 0;
    if (lane < nP) {
      const int qa = ROWS * lane, qb = qa + 1;
      const int ta = lrp[lo + qa], na = clampn(lrp[lo + qa + 1] - ta);
      if (ROWS == 2 && qb < nQ) {
        const int tb = lrp[lo + qb], nb = clampn(lrp[lo + qb + 1] - tb);
        int i = 0, j = 0;
        while (i < na || j < nb) {   // two ascending lists: size of the union
          const int a = i < na ? lci[ta + i] : 0x7fffffff, b = j < nb ? lci[tb + j] : 0x7fffffff;
          i += a <= b; j += b <= a; ++len;
        }
      } else {
        len = na;
      }
    }
    const int key = lane < nP ? (len << 6) | (63 - lane) : -1;
    const int mine = __shfl(key, g, 64);
    slot = __builtin_popcountll(__ballot(key > mine));
  }

  for (int r = 0; r < ROWS; ++r)
    for (int c = lane; c < nK; c += 64) { listed[r][c] = 0; partial[r][c] = 0; }
  __syncthreads();
  int p0[2] = {0, 0};
  for (int r = 0; r < ROWS; ++r) {
    const int qr = ROWS * g + r;
    if (qr >= nQ) continue;
    const int t0 = lrp[lo + qr], n = clampn(lrp[lo + qr + 1] - t0);
    for (int e = lane; e < n; e += 64) { const int c = lci[t0 + e]; if ((unsigned)c < (unsigned)nK) listed[r][c] = 1; }
    p0[r] = prp[lo + qr];
    const int np = clampn(prp[lo + qr + 1] - p0[r]);
    for (int e = lane; e < np; e += 64) { const int c = pci[p0[r] + e]; if ((unsigned)c < (unsigned)nK) { partial[r][c] = 1; pslot[r][c] = (unsigned short)e; } }
  }
  __syncthreads();

  uint64_t* blk = plan + ((int64_t)sample * nP + slot) * stride;
  int base = 0;
  for (int w = 0; w * 64 < nK; ++w) {
    const int c = 64 * w + lane;
    const bool in0 = c < nK && listed[0][c];
    const bool in1 = ROWS == 2 && c < nK && listed[ROWS - 1][c];
    const uint64_t any = __ballot(in0 || in1);
    if (in0 || in1) {
      const int pos = base + __builtin_popcountll(any & ((1ull << lane) - 1));
      const bool pa0 = in0 && partial[0][c], pa1 = in1 && partial[ROWS - 1][c];
      uint64_t word = (uint64_t)c | ((uint64_t)in0 << 16) | ((uint64_t)in1 << 17) | ((uint64_t)pa0 << 18) | ((uint64_t)pa1 << 19);
      if (pa0) word |= (uint64_t)pslot[0][c] << 32;
      if (pa1) word |= (uint64_t)pslot[ROWS - 1][c] << 48;
      blk[2 + pos] = word;
    }
    base += __builtin_popcountll(any);
  }
  if (lane == 0) {
    blk[0] = (uint64_t)g | ((uint64_t)base << 16);
    blk[1] = (uint64_t)(uint32_t)p0[0] | ((uint64_t)(uint32_t)p0[1] << 32);
  }
}

// Two query blocks per workgroup with the software-pipelined main loop (rings of three K and
// three V tiles: 48 KB of LDS).
template <int KIND, bool BF>
__global__ __launch_bounds__(256, 3) void block_attn_pipe_kernel(const AttnParams p) {
  STOF_ATTN_LDS_TILES;
  __shared__ __attribute__((aligned(1024))) unsigned char k_lds2[kTile];
  __shared__ __attribute__((aligned(1024))) unsigned char v_lds2[kTile];
  int bh, pair;
  RowPtrs<2> pre;
  pre.valid = false;
  if (p.balance) {
    balanced_group<KIND, 2>(p, bh, pair, pre);
  } else {
    const int vid = xcd_contiguous_id(p);
    if (vid >= p.total) return;
    bh = vid / p.nP;
    pair = zigzag(vid - bh * p.nP, bh, p.nP);
  }
  attn_group<KIND, 2, 1, true, BF>(p, bh, pair, pre, k_lds0, k_lds1, v_lds0, v_lds1, k_lds2, v_lds2);
}

// dst[r*(cols/64)+w] bit t = pred(src[r*ld + 64w + t]).
// Vector form: a lane loads 8 elements (16 B) and forms one byte of the word; the 8 lanes of a
// word merge their bytes with three lane exchanges and the first of them stores 8 B.  A
// wavefront covers 8 consecutive words (1 KB in, 64 B out) per load and issues kPackLoads loads
// before it looks at the first (one load per wave in flight kept the pass at the latency of its
// loads: 4096 x 4096 9.8 us); 16-byte aligned rows only.
constexpr int kPackLoads = 4;
__global__ __launch_bounds__(256) void pack_mask_bits_vec_kernel(const half_t* __restrict__ src,
                                                                 uint64_t* __restrict__ dst,
                                                                 int64_t rows, int64_t words_per_row,
                                                                 int64_t ld, int additive) {
  const int lane = threadIdx.x & 63;
  const int sub = lane & 7;
  const int64_t nwords = rows * words_per_row;
  const int64_t stride = (int64_t)gridDim.x * 32 * kPackLoads;
  for (int64_t w0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 8 * kPackLoads; w0 < nwords; w0 += stride) {
    half8_t x[kPackLoads];
#pragma unroll
    for (int u = 0; u < kPackLoads; ++u) {
      const int64_t w = w0 + 8 * u + (lane >> 3);
      const int64_t wc = w < nwords ? w : nwords - 1;   // (past the end: a valid address, the result is dropped)
      const int64_t r = wc / words_per_row;
      const int64_t cw = wc - r * words_per_row;
      x[u] = *reinterpret_cast<const half8_t*>(src + r * ld + cw * 64 + 8 * sub);
    }
#pragma unroll
    for (int u = 0; u < kPackLoads; ++u) {
      const int64_t w = w0 + 8 * u + (lane >> 3);
      uint32_t byte = 0;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (float)x[u][e];
        byte |= (uint32_t)(additive ? (f > -5000.f) : (f > 0.f)) << e;
      }
      uint32_t lo = sub < 4 ? byte << (8 * sub) : 0u, hi = sub < 4 ? 0u : byte << (8 * (sub - 4));
#pragma unroll
      for (int m = 1; m < 8; m <<= 1) {
        lo |= (uint32_t)__shfl_xor((int)lo, m, 64);
        hi |= (uint32_t)__shfl_xor((int)hi, m, 64);
      }
      if (sub == 0 && w < nwords) dst[w] = ((uint64_t)hi << 32) | lo;
    }
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
enum { kFormAuto = -1, kFormTwoRows = 0, kFormKeySplit = 1, kFormPipelined = 2 };

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

// Compute units of the current device, asked once per device (relaxed atomics: two threads that
// both find the slot empty store the same number).
int compute_units() {
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
  }
  return n;
}

int pick_form(int requested, int64_t two_row_groups, int nQ) {
  if (requested != kFormAuto) return requested;          // the caller's choice for this call
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

// plan_rows: query blocks per group of the plan in p.plan (0: none).  A plan laid out for the
// other group size is ignored (the kernel then walks the LUT itself).
template <int KIND, bool BF>
void launch_attn_as(AttnParams& p, int nQ, int64_t bh, int requested_form, int plan_rows, hipStream_t stream) {
  const int64_t two_row_groups = (int64_t)((nQ + kRowsPerGroup - 1) / kRowsPerGroup) * bh;
  const int form = pick_form(requested_form, two_row_groups, nQ);
  if (form == kFormKeySplit) {
    p.nP = nQ;
    p.total = (int)(nQ * bh);
    p.chunk = (p.total + 7) / 8;
    set_balance(p, kBalanceMaxGroupsKeySplit);
    if constexpr (KIND == kKindLut) {
      if (p.plan && plan_rows == 1) {
        hipLaunchKernelGGL((block_attn_fwd_kernel<KIND, 1, 2, BF, true>), dim3(p.chunk * 8), dim3(256), 0, stream, p);
        return;
      }
    }
    hipLaunchKernelGGL((block_attn_fwd_kernel<KIND, 1, 2, BF, false>), dim3(p.chunk * 8), dim3(256), 0, stream, p);
  } else {
    p.nP = (nQ + kRowsPerGroup - 1) / kRowsPerGroup;
    p.total = (int)two_row_groups;
    p.chunk = (p.total + 7) / 8;
    set_balance(p, kBalanceMaxGroupsTwoRows);
    if (form == kFormPipelined) {
      hipLaunchKernelGGL((block_attn_pipe_kernel<KIND, BF>), dim3(p.chunk * 8), dim3(256), 0, stream, p);
      return;
    }
    if constexpr (KIND == kKindLut) {
      if (p.plan && plan_rows == kRowsPerGroup) {
        hipLaunchKernelGGL((block_attn_fwd_kernel<KIND, kRowsPerGroup, 1, BF, true>), dim3(p.chunk * 8), dim3(128 * kRowsPerGroup), 0, stream, p);
        return;
      }
    }
    hipLaunchKernelGGL((block_attn_fwd_kernel<KIND, kRowsPerGroup, 1, BF, false>), dim3(p.chunk * 8), dim3(128 * kRowsPerGroup), 0, stream, p);
  }
}

template <int KIND>
void launch_attn(AttnParams& p, int nQ, int64_t bh, int requested_form, int dtype, int plan_rows, hipStream_t stream) {
  if (dtype == STOF_DTYPE_BF16) launch_attn_as<KIND, true>(p, nQ, bh, requested_form, plan_rows, stream);
  else launch_attn_as<KIND, false>(p, nQ, bh, requested_form, plan_rows, stream);
}

bool strides_ok(const int64_t s[3]) {
  return (s[0] % 8 == 0) && (s[1] % 8 == 0) && (s[2] % 8 == 0) && s[2] >= kD && s[2] < (1 << 20);
}

// K and V tiles are addressed with 32-bit byte offsets from the start of their (batch, head):
// the rows of one head must span less than 2^31 bytes.
bool span_ok(int64_t seq_len, int64_t row_stride) { return ((seq_len - 1) * row_stride + kD) * 2 < ((int64_t)1 << 31); }

}  // namespace

extern "C" int stof_attn_plan_rows(int batch_size, int head_num, int seq_len, int launch_form) {
  if (batch_size <= 0 || head_num <= 0 || seq_len <= 0 || seq_len % kBM != 0) return STOF_ERR_BAD_SHAPE;
  if (launch_form < kFormAuto || launch_form > kFormPipelined) return STOF_ERR_UNSUPPORTED;
  const int nQ = seq_len / kBM;
  const int64_t bh = (int64_t)batch_size * head_num;
  const int form = pick_form(launch_form, (int64_t)((nQ + kRowsPerGroup - 1) / kRowsPerGroup) * bh, nQ);
  if (form == kFormPipelined) return 0;
  return form == kFormKeySplit ? 1 : kRowsPerGroup;
}

extern "C" int64_t stof_attn_plan_bytes(int seq_len, int rows_per_group, int lut_batches) {
  if (seq_len <= 0 || seq_len % kBM != 0 || lut_batches <= 0 || (rows_per_group != 1 && rows_per_group != kRowsPerGroup)) return 0;
  const int nK = seq_len / kBN, nQ = seq_len / kBM;
  if (nK > kPlanMaxKeyBlocks) return 0;
  const int nP = (nQ + rows_per_group - 1) / rows_per_group;
  return (int64_t)lut_batches * nP * plan_stride_words(nK) * 8;
}

extern "C" int stof_attn_plan_build(const int32_t* part_row_ptr, const int32_t* part_col_idx,
                                    const int32_t* load_row_ptr, const int32_t* load_col_idx,
                                    int seq_len, int64_t lut_batch_stride, int lut_batches, int rows_per_group,
                                    void* plan, int64_t plan_bytes, void* stream) {
  if (!part_row_ptr || !load_row_ptr || !plan) return STOF_ERR_NULL_POINTER;
  const int64_t need = stof_attn_plan_bytes(seq_len, rows_per_group, lut_batches);
  if (need == 0) return STOF_ERR_UNSUPPORTED;
  if (plan_bytes < need) return STOF_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(plan) & 7) != 0) return STOF_ERR_MISALIGNED;
  const int nK = seq_len / kBN, nQ = seq_len / kBM;
  if (lut_batches > 1 && lut_batch_stride < nQ + 1) return STOF_ERR_BAD_LUT;
  const int nP = (nQ + rows_per_group - 1) / rows_per_group;
  if ((int64_t)lut_batches * nP > (int64_t)1 << 30) return STOF_ERR_BAD_SHAPE;
  const dim3 grid((unsigned)(lut_batches * nP));
  const int64_t bs = lut_batches > 1 ? lut_batch_stride : 0;
  if (rows_per_group == 1)
    hipLaunchKernelGGL((attn_plan_kernel<1>), grid, dim3(64), 0, (hipStream_t)stream, load_row_ptr, load_col_idx,
                       part_row_ptr, part_col_idx, bs, nQ, nK, nP, plan_stride_words(nK), (uint64_t*)plan);
  else
    hipLaunchKernelGGL((attn_plan_kernel<kRowsPerGroup>), grid, dim3(64), 0, (hipStream_t)stream, load_row_ptr, load_col_idx,
                       part_row_ptr, part_col_idx, bs, nQ, nK, nP, plan_stride_words(nK), (uint64_t*)plan);
  return stof_check_launch();
}

extern "C" int stof_block_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    const int32_t* full_row_ptr, const int32_t* full_col_idx,
    const int32_t* part_row_ptr, const int32_t* part_col_idx, const uint64_t* part_bitmask,
    const int32_t* load_row_ptr, const int32_t* load_col_idx,
    int block_m, int block_n, float softmax_scale,
    const int64_t q_strides[3], const int64_t k_strides[3],
    const int64_t v_strides[3], const int64_t out_strides[3],
    int batch_size, int seq_len, int head_num, int head_size, int dtype,
    int64_t lut_batch_stride, int launch_form, void* stream) {
  return stof_block_attn_fwd_planned(q, k, v, out, full_row_ptr, full_col_idx, part_row_ptr, part_col_idx, part_bitmask,
                                     load_row_ptr, load_col_idx, block_m, block_n, softmax_scale, q_strides, k_strides,
                                     v_strides, out_strides, batch_size, seq_len, head_num, head_size, dtype,
                                     lut_batch_stride, launch_form, nullptr, 0, 0, stream);
}

extern "C" int stof_block_attn_fwd_planned(
    const void* q, const void* k, const void* v, void* out,
    const int32_t* full_row_ptr, const int32_t* full_col_idx,
    const int32_t* part_row_ptr, const int32_t* part_col_idx, const uint64_t* part_bitmask,
    const int32_t* load_row_ptr, const int32_t* load_col_idx,
    int block_m, int block_n, float softmax_scale,
    const int64_t q_strides[3], const int64_t k_strides[3],
    const int64_t v_strides[3], const int64_t out_strides[3],
    int batch_size, int seq_len, int head_num, int head_size, int dtype,
    int64_t lut_batch_stride, int launch_form,
    const void* plan, int64_t plan_bytes, int plan_rows, void* stream) {
  if (launch_form < kFormAuto || launch_form > kFormPipelined) return STOF_ERR_UNSUPPORTED;
  if (dtype != STOF_DTYPE_F16 && dtype != STOF_DTYPE_BF16) return STOF_ERR_UNSUPPORTED;
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
  if (!span_ok(seq_len, k_strides[2]) || !span_ok(seq_len, v_strides[2])) return STOF_ERR_BAD_SHAPE;
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
  p.plan = nullptr; p.plan_stride = 0;
  if (plan) {
    const int64_t need = stof_attn_plan_bytes(seq_len, plan_rows, lut_batch_stride ? batch_size : 1);
    if (need == 0 || plan_bytes < need) return STOF_ERR_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(plan) & 7) != 0) return STOF_ERR_MISALIGNED;
    p.plan = (const uint64_t*)plan;
    p.plan_stride = plan_stride_words(seq_len / kBN);
  }
  launch_attn<kKindLut>(p, nQ, (int64_t)batch_size * head_num, launch_form, dtype, plan ? plan_rows : 0, (hipStream_t)stream);
  return stof_check_launch();
}

extern "C" int stof_rowwise_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    int kind, int is_causal, int bandwidth, const uint64_t* mask_bits,
    int batch_size, int seq_len, int head_num, int head_size, int dtype, int launch_form, void* stream) {
  if (launch_form < kFormAuto || launch_form > kFormPipelined) return STOF_ERR_UNSUPPORTED;
  if (dtype != STOF_DTYPE_F16 && dtype != STOF_DTYPE_BF16) return STOF_ERR_UNSUPPORTED;
  if (!q || !k || !v || !out) return STOF_ERR_NULL_POINTER;
  if (kind != STOF_ROW_FULL && kind != STOF_ROW_SLIDING && kind != STOF_ROW_MASK) return STOF_ERR_UNSUPPORTED;
  if (kind == STOF_ROW_MASK && !mask_bits) return STOF_ERR_NULL_POINTER;
  if (batch_size <= 0 || seq_len <= 0 || head_num <= 0 || head_size <= 0) return STOF_ERR_BAD_SHAPE;
  if (head_size != kD) return STOF_ERR_UNSUPPORTED;
  if (seq_len % kBM != 0) return STOF_ERR_BAD_SHAPE;
  if (kind == STOF_ROW_SLIDING && bandwidth <= 0) return STOF_ERR_BAD_SHAPE;
  if (!stof_aligned16(q) || !stof_aligned16(k) || !stof_aligned16(v) || !stof_aligned16(out)) return STOF_ERR_MISALIGNED;
  const int nQ = seq_len / kBM;
  if ((int64_t)nQ * batch_size * head_num > (int64_t)1 << 30 || !span_ok(seq_len, kD)) return STOF_ERR_BAD_SHAPE;
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
  p.plan = nullptr; p.plan_stride = 0;
  if (kind == STOF_ROW_MASK) launch_attn<kKindBits>(p, nQ, (int64_t)batch_size * head_num, launch_form, dtype, 0, (hipStream_t)stream);
  else launch_attn<kKindPred>(p, nQ, (int64_t)batch_size * head_num, launch_form, dtype, 0, (hipStream_t)stream);
  return stof_check_launch();
}

extern "C" int stof_pack_mask_bits(const void* src, uint64_t* dst, int64_t rows, int64_t cols, int64_t ld,
                                   int additive, void* stream) {
  if (!src || !dst) return STOF_ERR_NULL_POINTER;
  if (rows <= 0 || cols <= 0 || cols % 64 != 0 || ld < cols) return STOF_ERR_BAD_SHAPE;
  const int64_t nwords = rows * (cols / 64);
  if (ld % 8 == 0 && stof_aligned16(src)) {
    int64_t blocks = (nwords + 32 * kPackLoads - 1) / (32 * kPackLoads);
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
