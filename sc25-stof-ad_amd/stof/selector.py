"""Deterministic operator / launch-form selection for the attention path on MI355X.

Mirrors the interface of the reference's two-phase selector
(src/benchmk_attn_unified.py:33-163: ``GPUParams``, ``phase1_decision``, ``phase2_selection``,
``select_operator``) with the decisions re-derived for this implementation:

* phase 1 - which operator.  The reference sends sparse masks (valid-block ratio rho below
  tau = 1 / log2(S/16)^2) to its row-wise kernels because its block kernels waste work on
  mostly-empty tiles.  Here every operator runs on the same 64 x 64 tile engine and the
  block-wise operator skips empty tiles through the LUT, so block-wise is never slower per
  call; the row-wise operators differ only in needing no LUT (tile list from index
  arithmetic).  They are chosen when the LUT would not skip anything worth its indirection:
  rho at or above ``dense_tau`` of the tiles the predicate would visit anyway.
* phase 2 - which launch form of the kernel (the reference picks (num_warps, BLOCK_M, BLOCK_N)
  by an occupancy x parallelism score).  Tile shape is fixed at 64 x 64 with four wavefronts;
  the choice is between two query blocks per workgroup (K/V tiles shared, half the L2 -> LDS
  traffic) and the key split (one query block per workgroup, half-length chains), by how
  many workgroups a compute unit receives and how long the chains can be.  The same rule is
  built into ``stof_block_attn_fwd`` (its default); this module states it, explains it and
  ``apply`` runs the chosen operator with the chosen form as a per-call argument.

No measurement, search or autotuning takes place.
"""
from dataclasses import dataclass

__all__ = ["GPUParams", "Selection", "phase1_decision", "phase2_selection", "select_operator", "apply"]

BLOCK = 64


class GPUParams:
    """Machine description (reference: GPUParams, benchmk_attn_unified.py:33-51)."""

    def __init__(self, gpu_type="MI355X"):
        if gpu_type != "MI355X":
            raise ValueError(f"only MI355X is described here, got {gpu_type!r}")
        self.gpu_type = gpu_type
        self.cu_count = 256               # 8 XCDs x 32 compute units
        self.xcd_count = 8
        self.simd_per_cu = 4
        self.wave_size = 64
        self.lds_per_cu = 160 * 1024
        self.vgprs_per_simd_lane = 512
        self.max_waves_per_simd = 8
        self.l2_per_xcd = 4 * 1024 * 1024
        self.lds_per_group = 4 * BLOCK * 64 * 2      # K and V tiles, double buffered: 32 KB
        self.waves_per_group = 4
        self.resident_groups_per_cu = 4   # measured: the fifth 32 KB group does not become resident
        # launch-form rule (kKeySplitMaxGroupsPerCu / kKeySplitMinQueryBlocks in the kernel source)
        self.key_split_max_groups_per_cu = 2
        self.key_split_min_query_blocks = 4


@dataclass(frozen=True)
class Selection:
    operator: str          # "block-wise" | "row-wise"
    launch_form: str       # "two_rows" | "key_split"
    block_m: int
    block_n: int
    rho: float             # active tiles / tiles of the square
    groups_per_cu: float   # two-row workgroups per compute unit
    reason: str
    row_kind: str = "full"   # row-wise only: which of the reference's three row-wise operators
                             # (src/ops/package_op.py:11-48): "full" (dense / causal), "sliding", "mask"
    bandwidth: int = 0       # row_kind "sliding": the window (keys j > i - bandwidth)

    def __str__(self):
        if self.operator == "row-wise":
            return "row-wise"
        return f"block-wise {self.launch_form} m{self.block_m}n{self.block_n}"


def _active_blocks(load_row_ptr):
    last = load_row_ptr[-1] if load_row_ptr.dim() == 1 else load_row_ptr[0, -1]
    return int(last)


def phase1_decision(load_row_ptr, seq_len, is_causal=False, dense_tau=0.9, lut=None):
    """True -> block-wise (LUT) operator, False -> row-wise (predicate) operator.

    ``rho`` is the share of 64 x 64 tiles the LUT lists; the row-wise operators would visit
    every tile (the lower triangle when causal).  Block-wise unless the LUT lists at least
    ``dense_tau`` of those.  With the whole ``lut`` given (the seven tensors of
    ``get_sparse_storage``) the answer is exact instead of a density estimate: row-wise only if
    the LUT IS the predicate's pattern - every tile of the square listed and none partial
    (dense), or exactly the lower triangle listed, only the diagonal tiles partial and each of
    them the 64 x 64 lower triangle (causal) - so that ``rowwise_attn_full_op`` computes the
    same function; any other nearly-dense mask stays on the LUT, which keeps its partial tiles."""
    nq = seq_len // BLOCK
    visited = nq * (nq + 1) // 2 if is_causal else nq * nq
    if lut is None:
        return _active_blocks(load_row_ptr) < dense_tau * visited
    import torch
    frp, fci, prp, pci, pbm, lrp, lci = lut
    if lrp.dim() == 2:
        if lrp.shape[0] > 1:
            return True                              # per-sample masks: no single predicate
        lrp, prp = lrp[0], prp[0]
    rows = (lrp[1:] - lrp[:-1]).tolist()
    parts = (prp[1:] - prp[:-1]).tolist()
    if not is_causal:
        return not (rows == [nq] * nq and parts == [0] * nq)
    if rows != list(range(1, nq + 1)) or parts != [1] * nq or tuple(pbm.shape) != (nq, BLOCK, BLOCK):
        return True
    if pci.tolist() != list(range(nq)):
        return True
    tri = torch.tril(torch.ones(BLOCK, BLOCK, device=pbm.device)) > 0
    return not bool(((pbm == 0) == tri[None]).all())


def phase2_selection(gpu, seq_len, batch_size, head_num):
    """Launch form and the figures it rests on: (form, groups_per_cu, reason)."""
    nq = seq_len // BLOCK
    groups = ((nq + 1) // 2) * batch_size * head_num
    per_cu = groups / gpu.cu_count
    resident = gpu.resident_groups_per_cu
    if nq >= gpu.key_split_min_query_blocks and groups <= gpu.key_split_max_groups_per_cu * gpu.cu_count:
        return ("key_split", per_cu,
                f"{per_cu:.2f} two-row workgroups per compute unit (<= {gpu.key_split_max_groups_per_cu}, "
                f"{resident} fit, so twice as many still run as one round): run time is set by the longest chain "
                f"of key blocks, which the key split halves")
    if nq < gpu.key_split_min_query_blocks:
        why = f"chains of at most {nq} key blocks are too short for the split to pay"
    else:
        why = f"{per_cu:.2f} two-row workgroups per compute unit keep every SIMD busy; shared K/V tiles halve L2 -> LDS traffic"
    return ("two_rows", per_cu, why)


def _sliding_rows(nq, bandwidth, is_causal):
    """Key blocks per query block that the row-wise sliding operator visits: keys j > i - bandwidth,
    up to the diagonal block when causal, else to the end of the sequence."""
    rows = []
    for r in range(nq):
        first_key = BLOCK * r - bandwidth + 1
        lo = first_key // BLOCK if first_key > 0 else 0
        rows.append((r if is_causal else nq - 1) - lo + 1)
    return rows


def select_operator(gpu_params, load_row_ptr, batch_size, seq_len, head_num, is_causal=False, lut=None,
                    mask_kind=None, bandwidth=0):
    """Reference: select_operator(gpu_params, load_row_ptr, batch_size, seq_len, head_num),
    benchmk_attn_unified.py:157-163, which returns ``"block-wise warp{w}m{m}n{n}"`` or
    ``"row-wise"``; ``str()`` of the result here has the same two shapes.  Pass the whole
    ``lut`` as well to have "row-wise" returned only when the dense / causal row-wise operator
    computes exactly the LUT's mask (see ``phase1_decision``).

    ``mask_kind`` / ``bandwidth``: what the caller knows about the mask, as the reference's
    benchmark does by the mask's name: "sliding" with its bandwidth selects the row-wise
    sliding-window operator when the LUT lists exactly the tiles that window touches;
    ``load_row_ptr=None`` (no LUT at hand) selects the row-wise operator of the stated kind -
    "dense" / "causal" (full), "sliding", or "element" (the row-wise mask operator on ``row_mask``).
    The software-pipelined launch form is never selected: measured level with "two_rows" on grids
    of many rounds and behind it on single-round grids."""
    if seq_len % BLOCK:
        raise ValueError(f"seq_len ({seq_len}) must be a multiple of {BLOCK}")
    if mask_kind not in (None, "dense", "causal", "sliding", "element"):
        raise ValueError(f"mask_kind must be None, 'dense', 'causal', 'sliding' or 'element', got {mask_kind!r}")
    nq = seq_len // BLOCK
    form, per_cu, why = phase2_selection(gpu_params, seq_len, batch_size, head_num)
    # What the caller knows about the mask (the reference's benchmark knows its mask by name and
    # calls the matching row-wise operator, src/benchmk_attn_unified.py:396-407).  Every operator runs
    # on one tile engine here, so a row-wise operator is never faster per tile; it is the choice
    # where no LUT exists to drive the block-wise one, and where the LUT would list exactly the
    # tiles the operator's index predicate visits anyway (then it saves building LUT and plan).
    if load_row_ptr is None:
        if mask_kind is None:
            raise ValueError("without a LUT the mask kind must be given ('dense', 'causal', 'sliding' or 'element')")
        kind = {"dense": "full", "causal": "full", "sliding": "sliding", "element": "mask"}[mask_kind]
        if kind == "sliding" and bandwidth <= 0:
            raise ValueError("mask_kind='sliding' needs the bandwidth")
        return Selection("row-wise", form, BLOCK, BLOCK, float("nan"), per_cu, "no LUT given: row-wise by the stated mask kind; " + why,
                         row_kind=kind, bandwidth=int(bandwidth))
    rho = _active_blocks(load_row_ptr) / float(nq * nq)
    if mask_kind == "sliding" and bandwidth > 0:
        lrp = load_row_ptr if load_row_ptr.dim() == 1 else (load_row_ptr[0] if load_row_ptr.shape[0] == 1 else None)
        if lrp is not None and (lrp[1:] - lrp[:-1]).tolist() == _sliding_rows(nq, int(bandwidth), is_causal):
            return Selection("row-wise", form, BLOCK, BLOCK, rho, per_cu,
                             "the LUT lists exactly the tiles of the stated sliding window; " + why,
                             row_kind="sliding", bandwidth=int(bandwidth))
    if phase1_decision(load_row_ptr, seq_len, is_causal, lut=lut):
        return Selection("block-wise", form, BLOCK, BLOCK, rho, per_cu, why)
    return Selection("row-wise", form, BLOCK, BLOCK, rho, per_cu,
                     "the LUT lists nearly every tile the index predicate visits; " + why)


def apply(selection, q, k, v, lut=None, is_causal=False, out_layout="bshd", row_mask=None):
    """Run the selected operator in the selected launch form (passed per call, no process
    state involved) and return its result: ``[B,S,H*D]`` (``out_layout="bshd"``, the layout
    of the reference's row-wise operators) or ``[B,H,S,D]`` (``"bhsd"``, block-wise only).
    ``lut``: the seven LUT tensors, needed for "block-wise"; ``row_mask`` [S,S] of 0/1 for the
    row-wise element-mask operator."""
    from .ops import block_attn, rowwise_attn
    if selection.operator == "row-wise":
        if selection.row_kind == "mask" and row_mask is None:
            raise ValueError("the row-wise mask operator needs row_mask [S,S]")
        return rowwise_attn(selection.row_kind, q, k, v, is_causal, bandwidth=selection.bandwidth, row_mask=row_mask,
                            launch_form=selection.launch_form)
    if lut is None:
        raise ValueError("the block-wise operator needs the LUT")
    return block_attn(q, k, v, lut, selection.block_m, selection.block_n, out_layout=out_layout,
                      launch_form=selection.launch_form)
