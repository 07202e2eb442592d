// Block-masked multi-head attention for gfx950 (MI355X), head size 64, 64x64 LUT blocks.
//
// Replaces the 20 WMMA kernels + dispatcher of the reference
// (src/ops/src/block_attn_mask_cuda.cu:269-6322) with one kernel designed around the
// CDNA4 wavefront:
//
//  * one 64-lane wavefront (= one workgroup) owns one 64-row query block and walks the
//    LUT's key blocks for it; there is no cross-wave sharing, hence no workgroup barrier
//    that waits on another wave and no S/P/O traffic through LDS;
//  * scores are produced TRANSPOSED, S^T = K . Q^T, with v_mfma_f32_32x32x16_f16.  In the
//    32x32 accumulator layout a lane then holds 32 keys of ONE query (lane & 31), so the
//    online-softmax state (running max, running sum, rescale factor) is one scalar per
//    lane, the row reduction is a register loop plus a single exchange with lane ^ 32,
//    and the probabilities are already in the register layout the second product
//    O^T = V^T . P^T wants for its B operand - P never leaves registers;
//  * K is staged in LDS row-major (its contraction index d is contiguous in memory),
//    V is staged TRANSPOSED (contraction index = key must be contiguous per lane): each
//    lane gathers a 4-key x 8-channel patch with 16-byte loads and transposes it in
//    registers with v_perm_b32 before 8-byte LDS writes;
//  * masks: full tiles run mask-free, partial tiles test one bit per element from a
//    64-bit row mask (512 B per tile instead of the reference's 8 KB additive fp16 tile),
//    empty tiles are never visited;
//  * workgroup ids are remapped so that all query blocks of one (batch, head) run on one
//    XCD (K/V stay in that XCD's L2) and long LUT rows start first.
#include "stof_common.h"

namespace {

constexpr int kD = 64;        // head size
constexpr int kBM = 64;       // query rows per block
constexpr int kBN = 64;       // keys per block
constexpr int kLd = 72;       // LDS row pitch in halves: 64 + 8 pad (144 B) keeps the
                              // 16-byte fragment reads of 16 consecutive rows on distinct banks
constexpr float kMasked = -INFINITY;   // score given to a masked element

struct AttnParams {
  const half_t* q; const half_t* k; const half_t* v; half_t* out;
  const int32_t* frp; const int32_t* fci;
  const int32_t* prp; const int32_t* pci; const uint64_t* pbits;
  const int32_t* lrp; const int32_t* lci;
  int64_t qs[3], ks[3], vs[3], os[3];
  int64_t lut_bs;
  int B, S, H, nQ;
  int total, chunk;
  float c;  // softmax_scale * log2(e)
};

__device__ __forceinline__ floatx16 mfma32(half8_t a, half8_t b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// LUT cursor of one query block: yields (key block, bitmask slot or -1) in LOAD order,
// following the three-way rule of block_attn_mask_cuda.cu:3675-3700.
struct LutCursor {
  const int32_t* fci; const int32_t* pci; const int32_t* lci;
  int t, t_end, f, f_end, pp, pp_end;
  __device__ __forceinline__ bool next(int& col, int& slot) {
    while (t < t_end) {
      const int c = __builtin_amdgcn_readfirstlane(lci[t++]);
      if (f < f_end && __builtin_amdgcn_readfirstlane(fci[f]) == c) { ++f; col = c; slot = -1; return true; }
      if (pp < pp_end && __builtin_amdgcn_readfirstlane(pci[pp]) == c) { col = c; slot = pp++; return true; }
    }
    return false;
  }
};

__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void block_attn_fwd_kernel(const AttnParams p) {
  __shared__ __attribute__((aligned(16))) half_t Ks[kBN * kLd];
  __shared__ __attribute__((aligned(16))) half_t Vt[kD * kLd];

  const int lane = threadIdx.x;
  const int j32 = lane & 31;
  const int g = lane >> 5;

  // Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous range
  // of (batch, head, query block) so one head's K/V is read through a single L2.
  const int wg = blockIdx.x;
  const int vid = (wg & 7) * p.chunk + (wg >> 3);
  if (vid >= p.total) return;
  const int bh = vid / p.nQ;
  const int qi = p.nQ - 1 - (vid - bh * p.nQ);   // late (long, for causal-like masks) rows first
  const int b = bh / p.H;
  const int h = bh - b * p.H;

  const half_t* qb = p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)qi * kBM * p.qs[2];
  const half_t* kb = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vb = p.v + b * p.vs[0] + h * p.vs[1];
  half_t* ob = p.out + b * p.os[0] + h * p.os[1] + (int64_t)qi * kBM * p.os[2];

  // Q^T as the B operand: lane (n = query j32 of tile nt, k-group g) holds 8 consecutive d.
  half8_t qf[2][4];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
      qf[nt][ks] = *reinterpret_cast<const half8_t*>(qb + (int64_t)(32 * nt + j32) * p.qs[2] + 16 * ks + 8 * g);

  const int64_t lo = (int64_t)b * p.lut_bs;
  LutCursor cur;
  cur.fci = p.fci; cur.pci = p.pci; cur.lci = p.lci;
  cur.t = __builtin_amdgcn_readfirstlane(p.lrp[lo + qi]); cur.t_end = __builtin_amdgcn_readfirstlane(p.lrp[lo + qi + 1]);
  cur.f = __builtin_amdgcn_readfirstlane(p.frp[lo + qi]); cur.f_end = __builtin_amdgcn_readfirstlane(p.frp[lo + qi + 1]);
  cur.pp = __builtin_amdgcn_readfirstlane(p.prp[lo + qi]); cur.pp_end = __builtin_amdgcn_readfirstlane(p.prp[lo + qi + 1]);

  floatx16 oacc[2][2];   // [d tile][query tile]: O^T
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][j][r] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_run[2] = {0.f, 0.f};

  // staging lanes: 8 lanes cover one 128-byte row
  const int dc = lane & 7;     // 16-byte chunk (8 channels) within a row
  const int rq = lane >> 3;    // row (K) or key quad (V) handled by this lane, per round

  int col, slot;
  bool have = cur.next(col, slot);

  while (have) {
    // ---- K tile -> LDS (row-major); the V tile's loads stay in flight while S is computed
    {
      uint4 kr[8];
      const half_t* kt = kb + (int64_t)col * kBN * p.ks[2] + 8 * dc;
#pragma unroll
      for (int t = 0; t < 8; ++t) kr[t] = *reinterpret_cast<const uint4*>(kt + (int64_t)(8 * t + rq) * p.ks[2]);
#pragma unroll
      for (int t = 0; t < 8; ++t) *reinterpret_cast<uint4*>(&Ks[(8 * t + rq) * kLd + 8 * dc]) = kr[t];
    }
    uint4 vr[2][4];
    {
      const half_t* vt = vb + (int64_t)col * kBN * p.vs[2] + 8 * dc;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4)
          vr[t][c4] = *reinterpret_cast<const uint4*>(vt + (int64_t)(4 * (rq + 8 * t) + c4) * p.vs[2]);
    }
    __syncthreads();

    // ---- S^T = K . Q^T : sacc[nt][mt][r] = S[query 32nt+j32][key 32mt + 8(r/4) + 4g + r%4]
    floatx16 sacc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[i][j][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const half8_t a = *reinterpret_cast<const half8_t*>(&Ks[(32 * mt + j32) * kLd + 16 * ks + 8 * g]);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) sacc[nt][mt] = mfma32(a, qf[nt][ks], sacc[nt][mt]);
      }

    // ---- V tile -> LDS transposed.  This lane holds keys 4*qd .. 4*qd+3 (rows) x channels
    // 8*dc .. 8*dc+7; it writes, for each channel, the 4 keys as one 8-byte word at the
    // position the P.V A-operand read expects: key = 32mt + 16s + 8h + 4g' + c sits at
    // 32mt + 16s + 8g' + 4h + c, i.e. the two low bits of the quad index are swapped.
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int qd = rq + 8 * t;
      const int pq = (qd & ~3) | ((qd & 1) << 1) | ((qd >> 1) & 1);
      const uint4 a0 = vr[t][0], a1 = vr[t][1], a2 = vr[t][2], a3 = vr[t][3];
      const uint32_t v0[4] = {a0.x, a0.y, a0.z, a0.w};
      const uint32_t v1[4] = {a1.x, a1.y, a1.z, a1.w};
      const uint32_t v2[4] = {a2.x, a2.y, a2.z, a2.w};
      const uint32_t v3[4] = {a3.x, a3.y, a3.z, a3.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint2 ev, od;
        ev.x = __builtin_amdgcn_perm(v1[j], v0[j], 0x05040100u);
        ev.y = __builtin_amdgcn_perm(v3[j], v2[j], 0x05040100u);
        od.x = __builtin_amdgcn_perm(v1[j], v0[j], 0x07060302u);
        od.y = __builtin_amdgcn_perm(v3[j], v2[j], 0x07060302u);
        *reinterpret_cast<uint2*>(&Vt[(8 * dc + 2 * j) * kLd + 4 * pq]) = ev;
        *reinterpret_cast<uint2*>(&Vt[(8 * dc + 2 * j + 1) * kLd + 4 * pq]) = od;
      }
    }

    const int cur_slot = slot;
    const int cur_col = col;
    (void)cur_col;
    const bool have_next = cur.next(col, slot);
    __syncthreads();

    // ---- online softmax on S^T; one query per lane (and its partner lane ^ 32)
    half8_t pf[2][2][2];   // [query tile][key tile][half]: B operand of O^T = V^T . P^T
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      if (cur_slot >= 0) {
        const uint64_t bits = p.pbits[(int64_t)cur_slot * kBM + 32 * nt + j32];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const uint32_t w = (uint32_t)(bits >> (32 * mt)) >> (4 * g);
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (!((w >> (8 * (r >> 2) + (r & 3))) & 1u)) sacc[nt][mt][r] = kMasked;
        }
      }
      float mx = sacc[nt][0][0];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[nt][mt][r]);
      mx = fmaxf(mx, xchg32(mx));
      const float m_new = fmaxf(m_run[nt], mx);
      // A row that has seen no allowed key yet has m_new == -inf: subtract 0 instead, so
      // that its probabilities are exp2(-inf) = 0 and no inf - inf appears.
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run[nt] - m_sub) * p.c);
      const float mc = m_sub * p.c;
      float lsum = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[nt][mt][r], p.c, -mc));
          lsum += e;
          pf[nt][mt][r >> 3][r & 7] = (half_t)e;
        }
      l_run[nt] = l_run[nt] * alpha + lsum;   // per-lane partial sum; halves are added at the end
      m_run[nt] = m_new;
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][nt][r] *= alpha;
    }

    // ---- O^T += V^T . P^T
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          const half8_t a = *reinterpret_cast<const half8_t*>(&Vt[(32 * dt + j32) * kLd + 32 * mt + 16 * s2 + 8 * g]);
#pragma unroll
          for (int nt = 0; nt < 2; ++nt) oacc[dt][nt] = mfma32(a, pf[nt][mt][s2], oacc[dt][nt]);
        }
    have = have_next;
  }

  // ---- normalise and store: oacc[dt][nt][r] = O[query 32nt+j32][d = 32dt + 8(r/4) + 4g + r%4]
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const float l = l_run[nt] + xchg32(l_run[nt]);
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;   // no allowed key at all: zeros
    half_t* orow = ob + (int64_t)(32 * nt + j32) * p.os[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        half4_t o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) o4[e] = (half_t)(oacc[dt][nt][4 * q4 + e] * inv);
        *reinterpret_cast<half4_t*>(orow + 32 * dt + 8 * q4 + 4 * g) = o4;
      }
  }
}

// dst[r*(cols/64)+w] bit t = pred(src[r*ld + 64w + t]); one wavefront per 64-element word.
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

bool strides_ok(const int64_t s[3]) { return (s[0] % 8 == 0) && (s[1] % 8 == 0) && (s[2] % 8 == 0) && s[2] >= kD; }

}  // namespace

extern "C" int stof_block_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    const int32_t* full_row_ptr, const int32_t* full_col_idx,
    const int32_t* part_row_ptr, const int32_t* part_col_idx, const uint64_t* part_bitmask,
    const int32_t* load_row_ptr, const int32_t* load_col_idx,
    int block_m, int block_n, float softmax_scale,
    const int64_t q_strides[3], const int64_t k_strides[3],
    const int64_t v_strides[3], const int64_t out_strides[3],
    int batch_size, int seq_len, int head_num, int head_size,
    int64_t lut_batch_stride, void* stream) {
  if (!q || !k || !v || !out || !full_row_ptr || !part_row_ptr || !load_row_ptr ||
      !q_strides || !k_strides || !v_strides || !out_strides)
    return STOF_ERR_NULL_POINTER;
  // column lists / bitmask may legitimately be empty, but then must still be addressable
  // by the kernel's scalar loads only when their row ranges are non-empty; NULL is accepted.
  if (batch_size <= 0 || seq_len <= 0 || head_num <= 0 || head_size <= 0) return STOF_ERR_BAD_SHAPE;
  if (head_size != kD || block_m != kBM || block_n != kBN) return STOF_ERR_UNSUPPORTED;
  if (seq_len % kBM != 0) return STOF_ERR_BAD_SHAPE;
  const int nQ = seq_len / kBM;
  if (lut_batch_stride != 0 && lut_batch_stride < nQ + 1) return STOF_ERR_BAD_LUT;
  if (!load_col_idx) return STOF_ERR_NULL_POINTER;
  if (!stof_aligned16(q) || !stof_aligned16(k) || !stof_aligned16(v) || !stof_aligned16(out)) return STOF_ERR_MISALIGNED;
  if (!strides_ok(q_strides) || !strides_ok(k_strides) || !strides_ok(v_strides) || !strides_ok(out_strides))
    return STOF_ERR_MISALIGNED;
  const int64_t total64 = (int64_t)nQ * batch_size * head_num;
  if (total64 > (int64_t)1 << 30) return STOF_ERR_BAD_SHAPE;

  AttnParams p;
  p.q = (const half_t*)q; p.k = (const half_t*)k; p.v = (const half_t*)v; p.out = (half_t*)out;
  p.frp = full_row_ptr; p.fci = full_col_idx; p.prp = part_row_ptr; p.pci = part_col_idx;
  p.pbits = part_bitmask; p.lrp = load_row_ptr; p.lci = load_col_idx;
  for (int i = 0; i < 3; ++i) { p.qs[i] = q_strides[i]; p.ks[i] = k_strides[i]; p.vs[i] = v_strides[i]; p.os[i] = out_strides[i]; }
  p.lut_bs = lut_batch_stride;
  p.B = batch_size; p.S = seq_len; p.H = head_num; p.nQ = nQ;
  p.total = (int)total64;
  p.chunk = (p.total + 7) / 8;
  p.c = softmax_scale * 1.4426950408889634f;
  hipLaunchKernelGGL(block_attn_fwd_kernel, dim3(p.chunk * 8), dim3(64), 0, (hipStream_t)stream, p);
  return stof_check_launch();
}

extern "C" int stof_pack_mask_bits(const void* src, uint64_t* dst, int64_t rows, int64_t cols, int64_t ld,
                                   int additive, void* stream) {
  if (!src || !dst) return STOF_ERR_NULL_POINTER;
  if (rows <= 0 || cols <= 0 || cols % 64 != 0 || ld < cols) return STOF_ERR_BAD_SHAPE;
  const int64_t nwords = rows * (cols / 64);
  int64_t blocks = (nwords + 3) / 4;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(pack_mask_bits_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const half_t*)src, dst, rows, cols / 64, ld, additive);
  return stof_check_launch();
}
