/*
 * C ABI of libstof_hip.so - the gfx950 (MI355X) implementation of STOF's hot path:
 * block-masked multi-head attention driven by a full/partial/empty block LUT and
 * the fused encoder operators (GEMM+bias+activation, GEMM+bias+residual+LayerNorm,
 * bias+residual+LayerNorm).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; the library never
 *     allocates, frees or retains caller memory;
 *   - all activations are IEEE fp16 (two bytes; the attention entry points also take bfloat16);
 *     accumulation and statistics are fp32;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); launches
 *     are asynchronous, nothing synchronises;
 *   - every function returns 0 on success or a negative STOF_ERR_* code; no launch
 *     is made when an argument check fails.  stof_status_string() names a code.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   stof_block_attn_fwd        launch_block_attn_mask      src/ops/src/block_attn_mask.cpp:8-15,
 *                                                           src/ops/src/block_attn_mask_cuda.cu:6026-6322
 *   stof_attn_plan_*,
 *   stof_block_attn_fwd_planned  the LUT reads of the same kernels, block_attn_mask_cuda.cu:3590-3700
 *   stof_pack_mask_bits        (the fp16 additive blocks built at src/util/masks.py:159-166,
 *                               consumed at block_attn_mask_cuda.cu:3680-3698, and the fp16
 *                               row_mask of launcher_rowwise_attn_mask, rowwise_attn_mask_cuda.cu:89-101)
 *   stof_rowwise_attn_fwd      launcher_rowwise_attn_{full,sliding,mask}
 *                                                           src/ops/src/rowwise_attn_full.cpp:8-12,
 *                                                           rowwise_attn_sliding.cpp:8-12, rowwise_attn_mask.cpp:8-12
 *   stof_build_lut,
 *   stof_lut_additive_blocks   get_sparse_storage            src/util/masks.py:125-184 (the host loop :145-170)
 *   stof_retile_lut            the launcher's kernel selection by (BLOCK_M, BLOCK_N), block_attn_mask_cuda.cu:6064-6322
 *   stof_bias_res_ln           batched_bias_layer_norm_fused_kernel
 *                                                           src/triton_template/add_layernorm.py:19-107
 *   stof_gemm_bias_act         the first product + bias + GELU of triton_matmul_batch_kernel
 *                                                           src/triton_template/gemm_gemm.py:99-150
 *                              and matmul + bias (+ F.gelu)  src/benchmk_end2end.py:80-81
 *   stof_gemm_bias_act_splitk  the same interfaces (a second launch form: K split over workgroups)
 *   stof_gemm_bias_res_ln      batch_matmul_bias_layernorm_kernel
 *                                                           src/triton_template/gemm_add_layernorm.py:78-144
 *                              and matmul + bias + residual + F.layer_norm, src/benchmk_end2end.py:73-76
 *   stof_gemm_bias_res_ln_cluster  the same interfaces (a second launch form of the operator)
 *   stof_*_dt                  the entry points above with the element format as an argument (fp16 or bfloat16)
 */
#ifndef STOF_ABI_H
#define STOF_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define STOF_ABI_VERSION 4   /* 4: attention plan entry points, stof_retile_lut and the cluster form with a wait limit added, the two process-wide setters (attention launch form, cluster spin limit) removed - both are per-call arguments, the library keeps no mutable state; 3: split-K and element-format entry points (nothing removed or changed) */

enum {
  STOF_OK = 0,
  STOF_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
  STOF_ERR_BAD_SHAPE = -2,      /* a size is <= 0, not divisible as required, or too large */
  STOF_ERR_UNSUPPORTED = -3,    /* head size / block size / activation not implemented */
  STOF_ERR_MISALIGNED = -4,     /* pointer or stride breaks the 16-byte vector-access rule */
  STOF_ERR_LAUNCH = -5,         /* hipGetLastError() reported a failure after the launch */
  STOF_ERR_BAD_LUT = -6,        /* inconsistent LUT description (host-visible part) */
  STOF_ERR_TOO_LARGE = -7       /* the problem exceeds the fixed scratch of an entry point that allocates nothing */
};

/* activation selector of stof_gemm_bias_act */
enum { STOF_ACT_NONE = 0, STOF_ACT_GELU_ERF = 1, STOF_ACT_GELU_TANH = 2, STOF_ACT_RELU = 3 };

/* element format of q, k, v and out at the attention entry points */
enum { STOF_DTYPE_F16 = 0, STOF_DTYPE_BF16 = 1 };

/* launch form of the attention entry points */
enum { STOF_FORM_DEFAULT = -1, STOF_FORM_TWO_ROWS = 0, STOF_FORM_KEY_SPLIT = 1, STOF_FORM_PIPELINED = 2 };

/* rowwise front-end selector of stof_rowwise_attn_fwd */
enum { STOF_ROW_FULL = 0, STOF_ROW_SLIDING = 1, STOF_ROW_MASK = 2 };

int stof_abi_version(void);
const char* stof_status_string(int status);

/*
 * Block-masked multi-head attention, forward.
 *   out[b,h,i,:] = sum_j softmax_j( scale * q[b,h,i,:].k[b,h,j,:]  over allowed j ) v[b,h,j,:]
 * where the allowed (i,j) are described by the block LUT: the key blocks listed in LOAD for
 * query block i/block_m are visited; one that also appears in that row's PART list (at
 * position `slot` of the PART arrays) uses the 64-bit row masks
 * part_bitmask[slot*block_m + (i % block_m)] (bit j%block_n set = allowed), any other is
 * unmasked.  LOAD must be the union of FULL and PART and every row's LOAD and PART lists
 * must hold strictly ascending key-block indices, as get_sparse_storage builds them
 * (src/util/masks.py:149-166), which makes this the three-way rule of
 * block_attn_mask_cuda.cu:3675-3700; the FULL arrays are accepted for signature parity and
 * not read.  Query rows without any allowed key produce zeros.
 *
 * Tensors are addressed as base + b*stride_b + h*stride_h + s*stride_s + d (strides in
 * ELEMENTS, d contiguous), separately for q, k, v and out, so [B,H,S,D], [B,S,H,D] and
 * slices of a packed [B,S,3*H*D] projection are all accepted without a copy.  out may
 * alias q (the reference returns its result in q).
 *
 * LUT arrays are int32.  With lut_batch_stride == 0 the three row-pointer arrays have
 * S/block_m + 1 entries and are shared by every (b,h) as in the reference; otherwise
 * sample b uses row pointers at offset b*lut_batch_stride, whose values are absolute
 * offsets into the (concatenated) column lists and bitmask slots.  A column list or the bitmask
 * may be NULL when every row range over it is empty (no partial blocks; nothing allowed at all).
 *
 * Supported: D == 64, block_m == block_n == 64, S % 64 == 0 (the Python operator re-tiles LUTs
 * built with other block sizes to 64 x 64 before it calls this).  dtype: STOF_DTYPE_F16 (the
 * reference's only format) or STOF_DTYPE_BF16 for q, k, v and out alike; scores, softmax
 * statistics and the output accumulator are fp32 either way.
 *
 * launch_form is the per-call counterpart of the reference launcher's num_warps (its kernel
 * selection by (num_warps, BLOCK_M, BLOCK_N), block_attn_mask_cuda.cu:6064-6322):
 *   STOF_FORM_DEFAULT (-1) chosen by the library from the grid size;
 *   STOF_FORM_TWO_ROWS (0) two query blocks per workgroup, K/V tiles shared by four wavefronts
 *                          (large grids);
 *   STOF_FORM_KEY_SPLIT (1) one query block per workgroup, the 64 keys of every tile split over
 *                          two wavefront pairs whose partial results are merged at the end
 *                          (small grids).
 * Results are equal within rounding in every form; another value returns STOF_ERR_UNSUPPORTED.
 */
int stof_block_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    const int32_t* full_row_ptr, const int32_t* full_col_idx,
    const int32_t* part_row_ptr, const int32_t* part_col_idx, const uint64_t* part_bitmask,
    const int32_t* load_row_ptr, const int32_t* load_col_idx,
    int block_m, int block_n, float softmax_scale,
    const int64_t q_strides[3], const int64_t k_strides[3],
    const int64_t v_strides[3], const int64_t out_strides[3],
    int batch_size, int seq_len, int head_num, int head_size, int dtype,
    int64_t lut_batch_stride, int launch_form, void* stream);

/*
 * The walk of a LUT laid out ahead of time ("plan"), and stof_block_attn_fwd reading it.
 *
 * The reference's kernels read the LUT as it is: row pointers, then the row's column list, then
 * per key block a search of the PART list (block_attn_mask_cuda.cu:3590-3700).  Here a workgroup
 * owns one or two query blocks and visits the union of their key blocks; without a plan it reads
 * the row pointers of its whole head (to find its place in the order by row length), then the
 * column lists, and merges them - several dependent trips through memory before its first K/V
 * tile.  A plan holds, per LUT (per sample for per-sample LUTs) and per group in that order, the
 * finished walk: the workgroup's first load is its walk.  A LUT is usually built once and used for
 * every layer and step, so the plan is built once per LUT (one small launch) and kept beside it.
 *
 *   stof_attn_plan_rows   query blocks per workgroup (1 or 2) of the launch form that
 *                         stof_block_attn_fwd would use for this problem and launch_form - the
 *                         rows_per_group to build the plan with; 0 if that form reads no plan.
 *   stof_attn_plan_bytes  size of the plan in bytes; 0 = no plan for this shape (seq_len > 65536).
 *   stof_attn_plan_build  writes the plan for the LOAD / PART lists of a LUT (arguments as in
 *                         stof_block_attn_fwd; lut_batches = 1 for a shared LUT, else the batch
 *                         size with row pointers lut_batch_stride apart).  plan: device memory,
 *                         8-byte aligned, plan_bytes >= stof_attn_plan_bytes(...).
 *   stof_block_attn_fwd_planned  stof_block_attn_fwd plus the plan.  plan == NULL, or a plan whose
 *                         plan_rows is not what the launch form takes, runs exactly as
 *                         stof_block_attn_fwd does.  The plan must have been built from the same
 *                         LOAD / PART lists; results are bit-identical with and without it.
 */
int stof_attn_plan_rows(int batch_size, int head_num, int seq_len, int launch_form);
int64_t stof_attn_plan_bytes(int seq_len, int rows_per_group, int lut_batches);
int stof_attn_plan_build(const int32_t* part_row_ptr, const int32_t* part_col_idx,
                         const int32_t* load_row_ptr, const int32_t* load_col_idx,
                         int seq_len, int64_t lut_batch_stride, int lut_batches, int rows_per_group,
                         void* plan, int64_t plan_bytes, void* stream);
int stof_block_attn_fwd_planned(
    const void* q, const void* k, const void* v, void* out,
    const int32_t* full_row_ptr, const int32_t* full_col_idx,
    const int32_t* part_row_ptr, const int32_t* part_col_idx, const uint64_t* part_bitmask,
    const int32_t* load_row_ptr, const int32_t* load_col_idx,
    int block_m, int block_n, float softmax_scale,
    const int64_t q_strides[3], const int64_t k_strides[3],
    const int64_t v_strides[3], const int64_t out_strides[3],
    int batch_size, int seq_len, int head_num, int head_size, int dtype,
    int64_t lut_batch_stride, int launch_form,
    const void* plan, int64_t plan_bytes, int plan_rows, void* stream);

/*
 * Pack fp16 mask rows into bit rows: dst[r*(cols/64) + w] bit t = pred(src[r*ld + 64*w + t]).
 * additive != 0: src holds additive masks (0 = keep, -10000 = drop), pred(x) = x > -5000;
 * additive == 0: src holds 0/1 masks, pred(x) = x > 0 (the test of rowwise_attn_mask_cuda.cu:58).
 * The stack of partial blocks [n,64,64] is packed with rows = n*64, cols = 64, ld = 64.
 * cols % 64 == 0.  HBM-bound: 2*rows*cols bytes in, rows*cols/8 bytes out.
 */
int stof_pack_mask_bits(const void* src, uint64_t* dst, int64_t rows, int64_t cols, int64_t ld,
                        int additive, void* stream);

/*
 * Row-wise attention front-ends (dense/causal, sliding window, element mask) with the
 * reference's result layout out[B, S, H*D] (src/ops/package_op.py:11-48).
 *   kind STOF_ROW_FULL:    keys j <= (is_causal ? i : S-1)
 *   kind STOF_ROW_SLIDING: additionally j > i - bandwidth
 *   kind STOF_ROW_MASK:    additionally bit j of mask_bits[i*(S/64) + j/64] set
 * Unlike the reference kernels the softmax is max-subtracted (no overflow) and rows
 * without an allowed key produce zeros.  q, k, v contiguous [B,H,S,D], D == 64, S % 64 == 0.
 * dtype and launch_form as for stof_block_attn_fwd.
 */
int stof_rowwise_attn_fwd(
    const void* q, const void* k, const void* v, void* out,
    int kind, int is_causal, int bandwidth, const uint64_t* mask_bits,
    int batch_size, int seq_len, int head_num, int head_size, int dtype, int launch_form, void* stream);

/*
 * Block LUT of a dense 0/1 mask, built on the GPU: the classification loop of get_sparse_storage
 * (src/util/masks.py:145-170) as two launches (classify every tile in one pass over the mask,
 * then compact).  mask: seq_len x seq_len elements of elem_bytes (2: fp16, 4: fp32) at a row
 * pitch of ld elements - batch 0 of the reference's [B,S,S] tensor (:147).  A block_m x block_n
 * tile whose elements are all 1 is FULL, all 0 is absent, anything else PARTIAL (:149-166).
 * Outputs, all int32 device arrays owned by the caller:
 *   full/part/load_row_ptr [seq_len/block_m + 1]; full/part/load_col_idx with room for cap_full /
 *   cap_part / cap_load entries (seq_len/block_m * seq_len/block_n always suffices), ascending
 *   key-block indices per row, LOAD = FULL and PARTIAL merged;
 *   part_bitmask [cap_part][64] (optional, 64 x 64 blocks only): bit j of row i of PART slot s =
 *   key j allowed, the form stof_block_attn_fwd reads;
 *   counts[4] (optional): {entries in FULL, PART, LOAD; 1 if a capacity was too small (the lists are
 *   then truncated, the row pointers still exact)}.
 * workspace: stof_build_lut_workspace_bytes() bytes of device memory, 8-byte aligned, used as
 * scratch for the duration of the call (one class byte per tile, 512 B of bit rows per 64 x 64 tile, a
 * 2-byte count per tile and, in its last 16 bytes, the mask's non-zero count: stof_build_lut_nnz_offset).
 * block_m, block_n in {16, 32, 64, 128} dividing seq_len; mask 16-byte aligned, ld * elem_bytes
 * a multiple of 16.  HBM-bound: seq_len^2 * elem_bytes bytes read once.
 */
int64_t stof_build_lut_workspace_bytes(int seq_len, int block_m, int block_n);
/* Byte offset inside that workspace at which a call of stof_build_lut leaves the number of non-zero
 * mask elements as an int64 (counted in the same pass as the classification) and, in the 4 bytes
 * behind it, the reference's nnz figure (src/util/masks.py:137) as a float32: count / seq_len^2 * 100
 * in fp32 arithmetic; the last 16 bytes of the workspace. */
int64_t stof_build_lut_nnz_offset(int seq_len, int block_m, int block_n);
int stof_build_lut(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
                   int32_t* full_row_ptr, int32_t* full_col_idx,
                   int32_t* part_row_ptr, int32_t* part_col_idx,
                   int32_t* load_row_ptr, int32_t* load_col_idx,
                   uint64_t* part_bitmask, int32_t* counts,
                   int64_t cap_full, int64_t cap_part, int64_t cap_load,
                   void* workspace, int64_t workspace_bytes, void* stream);

/*
 * A LUT built with block_m x block_n blocks (each in {16, 32, 64, 128}) described again with the
 * 64 x 64 blocks stof_block_attn_fwd takes: what the reference's launcher does by selecting a kernel
 * per (BLOCK_M, BLOCK_N) (src/ops/src/block_attn_mask_cuda.cu:6064-6322) is done here by re-tiling
 * the LUT once.  Input: the FULL and PART lists of the source LUT (row pointers of seq_len/block_m + 1
 * entries - for one sample of a per-sample LUT, pass that sample's row pointers; their values may be
 * absolute offsets into concatenated lists) and its additive fp16 blocks part_block_mask
 * [n_part][block_m][block_n] (0 = allowed, -10000 = masked; may be NULL when there is no partial
 * block).  Output, workspace and counts as for stof_build_lut at 64 x 64 (part_bitmask required):
 * the lists are exactly those of get_sparse_storage(mask, 64, 64) on the mask the source LUT
 * encodes.  Two launches, no synchronisation; seq_len a multiple of 64, block_m and block_n.
 */
int stof_retile_lut(const int32_t* full_row_ptr, const int32_t* full_col_idx,
                    const int32_t* part_row_ptr, const int32_t* part_col_idx, const void* part_block_mask,
                    int block_m, int block_n, int seq_len,
                    int32_t* out_full_row_ptr, int32_t* out_full_col_idx,
                    int32_t* out_part_row_ptr, int32_t* out_part_col_idx,
                    int32_t* out_load_row_ptr, int32_t* out_load_col_idx,
                    uint64_t* out_part_bitmask, int32_t* counts,
                    int64_t cap_full, int64_t cap_part, int64_t cap_load,
                    void* workspace, int64_t workspace_bytes, void* stream);

/*
 * stof_build_lut without the workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The scratch is a fixed array in device memory that the
 * library holds per GPU until the process ends (8.05 MiB: class bytes, bit rows and per-tile counts for up to
 * stof_build_lut_static_max_tiles() = 16384 tiles, i.e. seq_len 8192 at 64 x 64 blocks); a
 * larger problem returns STOF_ERR_TOO_LARGE.  No hipMalloc / hipFree or allocating routine is
 * called.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 * streams, two host threads) race - serialise them, or give the overlapping ones a workspace
 * through stof_build_lut.  Nothing in the array has to start at zero (every byte a call reads it
 * has written itself).  Arguments and results are those of stof_build_lut.
 */
int64_t stof_build_lut_static_max_tiles(void);
int stof_build_lut_static(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
                          int32_t* full_row_ptr, int32_t* full_col_idx,
                          int32_t* part_row_ptr, int32_t* part_col_idx,
                          int32_t* load_row_ptr, int32_t* load_col_idx,
                          uint64_t* part_bitmask, int32_t* counts,
                          int64_t cap_full, int64_t cap_part, int64_t cap_load, void* stream);

/*
 * The reference's additive fp16 blocks for the PART list of a LUT:
 * part_block_mask[s] = -10000 * (1 - block.half()) (src/util/masks.py:159-166), fp16
 * [n_part, block_m, block_n], for PART slots 0 .. n_part-1 as stof_build_lut wrote them.
 */
int stof_lut_additive_blocks(const void* mask, int elem_bytes, int64_t ld, int seq_len, int block_m, int block_n,
                             const int32_t* part_row_ptr, const int32_t* part_col_idx, int64_t n_part,
                             void* part_block_mask, void* stream);

/*
 * y[m,:] = LayerNorm(x[m,:] + bias[:] + residual[m,:]) * gamma + beta     (fp32 statistics)
 * bias, residual, gamma, beta may be NULL (treated as 0, 0, 1, 0); mean/rstd (fp32 [M]) may
 * be NULL.  N % 8 == 0, N <= 8192, rows are N contiguous elements at ld_* element pitch.
 * HBM-bound: 2*M*N bytes per operand that is present.
 */
int stof_bias_res_ln(const void* x, const void* bias, const void* residual,
                     const void* gamma, const void* beta, void* y,
                     float* mean, float* rstd,
                     int64_t M, int64_t N, float eps, void* stream);

/*
 * C[M,N] = act( A[M,K] @ W^T + bias[N] ) with W given as Wt[N,K] (K contiguous, the
 * nn.Linear orientation).  A rows at pitch lda, C rows at pitch ldc (elements).
 * K % 64 == 0, N % 8 == 0, lda % 8 == 0, ldc % 8 == 0; M arbitrary.  bias may be NULL.
 */
int stof_gemm_bias_act(const void* A, const void* Wt, const void* bias, void* C,
                       int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                       int act, void* stream);

/*
 * The same operator (src/triton_template/gemm_gemm.py:99-150, src/benchmk_end2end.py:80-81) with
 * the K dimension split over `splits` workgroups per tile of 64 rows x 128 features, for shapes
 * with few output tiles and a long K (a BERT-base FFN-out product at 512 tokens is 48 tiles and
 * K = 3072: one workgroup per tile leaves four compute units in five without work).  Each
 * workgroup leaves fp32 partial sums in `workspace`; the one that finishes last adds them in the
 * order of the splits (so the result does not depend on the order of arrival), applies bias and
 * activation and writes C.  Arguments and rules as stof_gemm_bias_act, plus:
 *   splits      2 .. 8 (fewer are used when K / 64 has fewer than that many k-tiles);
 *   workspace   at least stof_gemm_bias_act_splitk_workspace_bytes(M, N, splits) bytes, 16-byte
 *               aligned, ZERO at first use; every call leaves its counters zero again, so one
 *               workspace serves any sequence of calls on one stream (calls that overlap in time
 *               need workspaces of their own).  At most 4096 tiles (else STOF_ERR_UNSUPPORTED).
 * stof_gemm_bias_act_splitk_plan returns the number of splits this library would use for a shape,
 * 1 where stof_gemm_bias_act is the form to call (its rule: the plain form would run at most 128
 * tiles of 128 x 128, the split grid stays within 256 workgroups and 3 splits, and every split
 * keeps K >= 768; or 129 .. 192 tiles of 128 x 128 with K >= 3072: 2 splits).
 */
int stof_gemm_bias_act_splitk_plan(int64_t M, int64_t N, int64_t K);
int64_t stof_gemm_bias_act_splitk_workspace_bytes(int64_t M, int64_t N, int splits);
int stof_gemm_bias_act_splitk(const void* A, const void* Wt, const void* bias, void* C,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                              int act, int splits, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Y[M,H] = act( X[M,K] @ W1^T + b1[F] ) @ W2^T (+ b2[H]) in ONE launch, W1 given as W1t[F,K] and W2
 * as W2t[H,F] (nn.Linear orientation); the [M,F] intermediate is rounded to fp16 and stays on
 * chip.  Replaces triton_matmul_batch (src/triton_template/gemm_gemm.py:99-174; b2 is an
 * addition for the encoder's second FFN bias, NULL gives the reference's result).  Meant for
 * small M (<= ~1024 rows), where two separate GEMM launches are latency-bound.
 * K % 64 == 0, F % 128 == 0, H % 128 == 0, ldx % 8 == 0, ldy % 4 == 0; b1, b2 may be NULL.
 * workspace: stof_gemm_act_gemm_workspace_bytes(M, H) bytes of device memory (16-byte aligned)
 * that hold ZEROS at the first call; every call leaves them zero again, so one buffer serves
 * any number of calls that do not overlap in time (calls sharing a workspace on different
 * streams race).  The contributions of the F / 128 chunks are added in fp32 with atomic adds,
 * so the last bits of the fp32 sums depend on arrival order.
 */
int64_t stof_gemm_act_gemm_workspace_bytes(int64_t M, int64_t H);
int stof_gemm_act_gemm(const void* X, const void* W1t, const void* b1, const void* W2t, const void* b2,
                       void* Y, int64_t M, int64_t K, int64_t F, int64_t H, int64_t ldx, int64_t ldy,
                       int act, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * C[M,N] = LayerNorm( A[M,K] @ W^T + bias[N] + residual[M,N] ) * gamma + beta, the whole
 * row of N owned by one workgroup so the pre-normalisation values never reach HBM.
 * N in {256, 512, 768, 1024}; K % 32 == 0.  bias / residual / gamma / beta may be NULL.
 */
int stof_gemm_bias_res_ln(const void* A, const void* Wt, const void* bias, const void* residual,
                          const void* gamma, const void* beta, void* C,
                          int64_t M, int64_t N, int64_t K, float eps, void* stream);

/*
 * The same operator as stof_gemm_bias_res_ln (gemm_add_layernorm.py:78-144; benchmk_end2end.py:73-76,
 * 83-86) on 128 x 128 tiles: the N / 128 workgroups that share a block of 128 token rows
 * exchange per-row statistics (mean and sum of squared deviations of their 128 columns) through
 * `workspace`, so the pre-normalisation values still never reach HBM while the grid is N / 128
 * times larger.  The form for token counts at which one workgroup per 64 rows leaves compute
 * units idle (8192 tokens at hidden 768 / 1024).
 * N a multiple of 128 from 256 to 1024; K % 64 == 0; M <= 2^21; A rows at pitch lda, residual rows at pitch
 * ldr, C rows at pitch ldc (elements, multiples of 8); A, Wt, residual, C 16-byte aligned.
 * bias / residual / gamma / beta may be NULL.
 * workspace: stof_gemm_bias_res_ln_cluster_workspace_bytes(M, N) bytes (0 = shape not supported)
 * of device memory, 16-byte aligned, that hold ZEROS at the first call; every call leaves them
 * zero again, so one buffer serves any sequence of calls, of any shapes, that do not overlap in
 * time (calls sharing a workspace on different streams race).  The first 4 bytes are an error
 * word: a workgroup whose bounded wait for its partners ran out sets it to 1 (the output is
 * then invalid); it is never set in normal operation and stays set until the caller clears it.
 * The launch is at most as many workgroups as run at once (two per compute unit; the runtime's
 * occupancy figure for the kernel is asked, and a device that holds less than one row block's
 * workgroups per XCD returns STOF_ERR_UNSUPPORTED); each takes its tiles one after another.  They
 * all run at once when the device is otherwise free.  A kernel of another stream or process that
 * keeps compute units occupied for longer than the wait lasts (about 0.1 s) can keep part of the
 * grid from starting and make the waits of the rest run out: where such kernels share the
 * device, read the error word after the work that used this form (any later point will do: the
 * word stays set), or use stof_gemm_bias_act + stof_bias_res_ln instead.
 */
int64_t stof_gemm_bias_res_ln_cluster_workspace_bytes(int64_t M, int64_t N);
/* stof_gemm_bias_res_ln_cluster_dt with the length of the bounded wait as an argument: spin_limit polls
 * (0 = the default of 2^18, about a tenth of a second) before a wave gives up and sets the error
 * word.  With a limit of 1 a launch ends normally with the error word set: the way to test a
 * caller's handling of that word without disturbing the device. */
int stof_gemm_bias_res_ln_cluster_bounded(const void* A, const void* Wt, const void* bias, const void* residual,
                                          const void* gamma, const void* beta, void* C,
                                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldr, int64_t ldc,
                                          float eps, void* workspace, int64_t workspace_bytes, int dtype,
                                          int spin_limit, void* stream);
int stof_gemm_bias_res_ln_cluster(const void* A, const void* Wt, const void* bias, const void* residual,
                                  const void* gamma, const void* beta, void* C,
                                  int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldr, int64_t ldc,
                                  float eps, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * The four entry points above for tensors in either 16-bit format: the same arguments plus
 * dtype = STOF_DTYPE_F16 (what the functions without the suffix pass) or STOF_DTYPE_BF16, before
 * `stream`.  With bfloat16 every activation, weight, bias, gamma / beta and output tensor is
 * bfloat16, the products run on v_mfma_f32_32x32x16_bf16 and accumulation, statistics and
 * workspaces stay fp32.  (The reference computes in fp16 only; bfloat16 is an addition behind
 * the same operators.  stof_gemm_bias_res_ln and stof_gemm_act_gemm take fp16 only.)
 */
int stof_bias_res_ln_dt(const void* x, const void* bias, const void* residual,
                        const void* gamma, const void* beta, void* y,
                        float* mean, float* rstd,
                        int64_t M, int64_t N, float eps, int dtype, void* stream);
int stof_gemm_bias_act_dt(const void* A, const void* Wt, const void* bias, void* C,
                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                          int act, int dtype, void* stream);
int stof_gemm_bias_act_splitk_dt(const void* A, const void* Wt, const void* bias, void* C,
                                 int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                                 int act, int splits, void* workspace, int64_t workspace_bytes,
                                 int dtype, void* stream);
int stof_gemm_bias_res_ln_cluster_dt(const void* A, const void* Wt, const void* bias, const void* residual,
                                     const void* gamma, const void* beta, void* C,
                                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldr, int64_t ldc,
                                     float eps, void* workspace, int64_t workspace_bytes, int dtype, void* stream);

/*
 * Measurement probes (no counterpart in the reference; used by bench.py, not by any operator).
 * stof_device_compute_units: compute units of the current device (hipDeviceAttributeMultiprocessorCount),
 * or a negative status.  stof_probe_clock: one wavefront spins for `iters` x 16 dependent adds between
 * two readings of the shader cycle counter and of the constant 100 MHz counter and writes
 * {shader cycles, 10 ns ticks, scratch} to out3 (device memory, three 8-byte words): shader clock =
 * out3[0] / out3[1] * 100 MHz.  Launched on a second stream while other kernels run, it reads the
 * clock the chip holds under that load.
 */
int stof_device_compute_units(void);
int stof_probe_clock(unsigned long long* out3, int iters, void* stream);
/*
 * The arithmetic of one step of the attention loop (per wavefront 32 queries x 64 keys at head size
 * 64: 16 MFMA 32x32x16, 32 multiply-adds, 32 exp2, 16 converts, 16 packed adds, 16 max3) with no
 * memory access, LDS access or barrier, run for `steps` steps by waves_per_simd (1 .. 4) wavefronts
 * on every SIMD of the device.  parts: 1 = the MFMAs only, 2 = the vector arithmetic only, 3 = both.
 * The launch's duration / (steps * waves_per_simd) is the time one SIMD needs per wave-step of this
 * mix: the ceiling of the loop before loads, LDS reads, barriers, masks and the walk.  out3 as for
 * stof_probe_clock (first wavefront of the launch; out3[2] = steps); sink256: 256 floats of device
 * memory, never written in practice.
 */
int stof_probe_issue_mix(int parts, int waves_per_simd, int steps, unsigned long long* out3, float* sink256, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* STOF_ABI_H */
