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
  built into ``stof_block_attn_fwd``; this module states it, explains it and lets a caller
  apply it explicitly through ``apply``.

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

    def __str__(self):
        if self.operator == "row-wise":
            return "row-wise"
        return f"block-wise {self.launch_form} m{self.block_m}n{self.block_n}"


def _active_blocks(load_row_ptr):
    last = load_row_ptr[-1] if load_row_ptr.dim() == 1 else load_row_ptr[0, -1]
    return int(last)


def phase1_decision(load_row_ptr, seq_len, is_causal=False, dense_tau=0.9):
    """True -> block-wise (LUT) operator, False -> row-wise (predicate) operator.

    ``rho`` is the share of 64 x 64 tiles the LUT lists; the row-wise operators would visit
    every tile (the lower triangle when causal).  Block-wise unless the LUT lists at least
    ``dense_tau`` of those."""
    nq = seq_len // BLOCK
    visited = nq * (nq + 1) // 2 if is_causal else nq * nq
    return _active_blocks(load_row_ptr) < dense_tau * visited


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


def select_operator(gpu_params, load_row_ptr, batch_size, seq_len, head_num, is_causal=False):
    """Reference: select_operator(gpu_params, load_row_ptr, batch_size, seq_len, head_num),
    benchmk_attn_unified.py:157-163, which returns ``"block-wise warp{w}m{m}n{n}"`` or
    ``"row-wise"``; ``str()`` of the result here has the same two shapes."""
    if seq_len % BLOCK:
        raise ValueError(f"seq_len ({seq_len}) must be a multiple of {BLOCK}")
    nq = seq_len // BLOCK
    rho = _active_blocks(load_row_ptr) / float(nq * nq)
    form, per_cu, why = phase2_selection(gpu_params, seq_len, batch_size, head_num)
    if phase1_decision(load_row_ptr, seq_len, is_causal):
        return Selection("block-wise", form, BLOCK, BLOCK, rho, per_cu, why)
    return Selection("row-wise", form, BLOCK, BLOCK, rho, per_cu,
                     "the LUT lists nearly every tile the index predicate visits; " + why)


def apply(selection):
    """Force the selected launch form for the calls that follow (``"auto"`` applies the same
    rule inside the library)."""
    from .ops import set_attention_launch_form
    set_attention_launch_form(selection.launch_form)
