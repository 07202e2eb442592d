"""Attention operators: the reference's ``src/ops/package_op.py`` API on the HIP library.

``block_attn_mask_op`` and the three ``rowwise_attn_*_op`` keep the reference's call
signatures, tensor layouts and return conventions (src/ops/package_op.py:10-74):

* block op: q, k, v ``[B,H,S,D]`` fp16, the seven LUT tensors of ``get_sparse_storage``,
  ``BLOCK_M, BLOCK_N, num_warps``; the result overwrites ``q`` and ``q`` is returned;
* row-wise ops: a new zero-initialised ``[B, S, H*D]`` tensor is returned.

``block_attn`` is the functional form underneath (separate output, strided inputs, output
layout choice, optional per-sample LUT).  Everything runs in libstof_hip.so; there is no
PyTorch fallback - a missing library or an unsupported configuration raises ``StofError``.
"""
import math

import torch
from torch.autograd import Function

from . import _lib
from ._cache import (BITS_ATTR as _BITS_ATTR, DEVICE_BUILT_ATTR as _DEVICE_BUILT_ATTR, LUT_OK_ATTR as _LUT_OK_ATTR,
                     content_key as _content_key)
from ._lib import StofError, check, strides3

__all__ = ["block_attn", "BoundAttention", "block_attn_packed_qkv", "rowwise_attn", "block_attn_mask_op", "rowwise_attn_full_op", "rowwise_attn_sliding_op",
           "rowwise_attn_mask_op", "pack_mask_bits", "set_attention_launch_form", "StofError"]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device=None):
    """Raw handle of torch's current stream on ``device`` (a torch.device) or the current device."""
    if _raw_stream is not None and device is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _ptr(t):
    return t.data_ptr() if t is not None and t.numel() > 0 else None


def _require(cond, msg):
    if not cond:
        raise StofError(msg)


_DTYPES = {torch.float16: 0, torch.bfloat16: 1}   # STOF_DTYPE_*
_LAUNCH_FORMS = {None: -1, "default": -1, "auto": -1, "two_rows": 0, "key_split": 1, "pipelined": 2}


def _form(launch_form):
    _require(launch_form in _LAUNCH_FORMS,
             f"launch form must be one of 'default', 'two_rows', 'key_split', 'pipelined', got {launch_form!r}")
    f = _LAUNCH_FORMS[launch_form]
    return _default_form if f < 0 and launch_form != "auto" else f


_default_form = -1


def set_attention_launch_form(form="auto"):
    """DEFAULT launch form of the attention operators of this module, used by calls that do not
    name one: ``"auto"`` (the library chooses by grid size), ``"two_rows"`` (two query blocks per
    workgroup, for large grids), ``"key_split"`` (one query block per workgroup with the keys of
    each tile split over two wavefront pairs, for small grids) or ``"pipelined"``.  The reference
    selects its kernel per call with ``num_warps`` (src/ops/src/block_attn_mask_cuda.cu:6064-6322);
    the per-call counterpart here is the ``launch_form`` argument of ``block_attn`` and of the
    row-wise operators' functional form.  The default lives in this Python module (the library
    keeps no state: every C-ABI call names its form).  Results agree within rounding in every form."""
    global _default_form
    _require(form in ("auto", "two_rows", "key_split", "pipelined"),
             f"launch form must be 'auto', 'two_rows', 'key_split' or 'pipelined', got {form!r}")
    _default_form = _LAUNCH_FORMS[form]


def pack_mask_bits(src, additive):
    """fp16 ``[..., rows, cols]`` mask -> uint64-as-int64 ``[..., rows, cols/64]`` bit rows.
    additive=True: 0 keeps / -10000 drops (the LUT's partial blocks);
    additive=False: value > 0 keeps (the row-wise op's ``row_mask``)."""
    _require(src.is_cuda and src.dtype == torch.float16, "mask must be a CUDA fp16 tensor")
    src = src.contiguous()
    cols = src.shape[-1]
    _require(cols % 64 == 0, f"mask columns ({cols}) must be a multiple of 64")
    rows = src.numel() // cols
    dst = torch.empty(src.shape[:-1] + (cols // 64,), dtype=torch.int64, device=src.device)
    check(_lib.lib().stof_pack_mask_bits(src.data_ptr(), dst.data_ptr(), rows, cols, cols,
                                         1 if additive else 0, _stream(src.device)), "stof_pack_mask_bits")
    return dst


def _drop_caches(lut):
    """Forget what was derived from a LUT's tensors (``revalidate=True``).  Tensors the library
    itself produced on the device (masks.build_lut_device, a re-tiled LUT) keep their bit rows
    and their "in order" mark: those ARE the LUT's content there - the placeholder block mask
    they hang on holds nothing to derive them from again."""
    for t in lut:
        keep = (_BITS_ATTR, _LUT_OK_ATTR) if getattr(t, _DEVICE_BUILT_ATTR, False) else ()
        for attr in (_BITS_ATTR, _LUT_OK_ATTR, _LUT64_ATTR, _LUT_READY_ATTR):
            if attr in keep:
                continue
            if hasattr(t, attr):
                try:
                    delattr(t, attr)
                except AttributeError:
                    pass


def _packed_partial_bits(part_block_mask):
    """Bit rows of the LUT's partial blocks, packed once per tensor object and content
    version and kept on the tensor itself."""
    key = _content_key(part_block_mask)
    cached = getattr(part_block_mask, _BITS_ATTR, None)
    if cached is not None and cached[0] == key:
        return cached[1]
    pbm = part_block_mask
    _require(pbm.dim() == 3, "part_block_mask must be [n_part, BLOCK_M, BLOCK_N]")
    # The kernel applies element masks as bits; additive values other than 0 / -10000
    # (or the all-ones dummy block of an LUT without partial tiles) cannot be represented.
    ok = ((pbm == 0) | (pbm == -10000.0)).all() | ((pbm == 1).all() & (pbm.shape[0] == 1))
    _require(bool(ok), "part_block_mask must hold only 0 and -10000 (get_sparse_storage's encoding)")
    bits = pack_mask_bits(pbm, additive=True)
    try:
        setattr(part_block_mask, _BITS_ATTR, (key, bits))
    except AttributeError:
        pass
    return bits


def _check_lut_order(lrp, lci, prp, pci, n_cols):
    """The kernel walks each row's LOAD and PART lists as ascending sets (that is how
    get_sparse_storage emits them); verify once per column-list tensor and content version."""
    cached = getattr(lci, _LUT_OK_ATTR, None)
    key = tuple(_content_key(t) for t in (lci, pci, lrp, prp))
    if cached == key:
        return
    for name, rp, ci in (("load", lrp, lci), ("part", prp, pci)):
        if ci.numel() == 0:
            continue
        flat = rp.reshape(-1, rp.shape[-1]).long()
        used = int(flat.max())
        _require(0 <= used <= ci.numel(), f"{name}_row_ptr points past the end of {name}_col_idx")
        ci = ci[:used]                       # (lists kept at full capacity: the tail is unused)
        if used == 0:
            continue
        ok = bool((ci >= 0).all()) and bool((ci < n_cols).all())
        if ci.numel() > 1:
            inc = ci[1:] > ci[:-1]
            starts = torch.zeros(ci.numel(), dtype=torch.bool, device=ci.device)
            idx = flat[:, :-1].reshape(-1)
            idx = idx[idx < ci.numel()]
            starts[idx] = True               # a row boundary may go down
            ok = ok and bool((inc | starts[1:]).all())
        ok = ok and bool((flat[:, 1:] >= flat[:, :-1]).all()) and int(flat.max()) <= ci.numel()
        _require(ok, f"{name}_row_ptr / {name}_col_idx must describe rows of strictly ascending key-block "
                     f"indices in [0, {n_cols}) (get_sparse_storage's layout)")
    try:
        setattr(lci, _LUT_OK_ATTR, key)
    except AttributeError:
        pass


_LUT64_ATTR = "_stof_lut_at_64"


def _lut_at_64(lut, S, block_m, block_n):
    """The same mask described with 64 x 64 blocks, for a LUT built with another block size
    (the reference's kernels cover BLOCK_M / BLOCK_N of 16..128,
    src/ops/src/block_attn_mask_cuda.cu:6064-6322; the kernel here has one tile shape).  The
    library re-tiles the LUT on the device (stof_retile_lut: full source block -> ones, partial
    -> the bits of its additive values, absent -> zeros, classified again at 64 x 64); the
    attention result depends on the mask only, so this changes nothing but the tiling.  Shared
    and per-sample LUTs alike (a per-sample LUT is re-tiled sample by sample).  Done once per
    LUT (kept on the LOAD column tensor, keyed by the tensors' content versions)."""
    frp, fci, prp, pci, pbm, lrp, lci = lut
    key = tuple(_content_key(t) for t in lut) + (block_m, block_n)
    cached = getattr(lci, _LUT64_ATTR, None)
    if cached is not None and cached[0] == key:
        return cached[1]
    _require(block_m in (16, 32, 64, 128) and block_n in (16, 32, 64, 128),
             f"LUT block sizes must be 16, 32, 64 or 128, got {block_m} x {block_n}")
    n_part = int(prp.reshape(-1)[-1])
    _require(n_part == 0 or (pbm.dim() == 3 and tuple(pbm.shape[-2:]) == (block_m, block_n) and pbm.shape[0] >= n_part),
             f"part_block_mask must hold {n_part} blocks of {block_m} x {block_n}")
    dev = lrp.device
    lib = _lib.lib()
    n64 = S // 64
    tiles = n64 * n64
    pbm_c = pbm.contiguous() if n_part else None
    ws = torch.empty(lib.stof_build_lut_workspace_bytes(S, 64, 64), dtype=torch.uint8, device=dev)
    frp2, prp2 = frp.reshape(-1, frp.shape[-1]), prp.reshape(-1, prp.shape[-1])
    per_sample = []
    for b in range(frp2.shape[0]):
        i32 = lambda k: torch.empty(k, dtype=torch.int32, device=dev)
        o_frp, o_prp, o_lrp = i32(n64 + 1), i32(n64 + 1), i32(n64 + 1)
        o_fci, o_pci, o_lci, counts = i32(tiles), i32(tiles), i32(tiles), i32(4)
        o_bits = torch.empty((tiles, 64), dtype=torch.int64, device=dev)
        check(lib.stof_retile_lut(frp2[b].data_ptr(), _ptr(fci), prp2[b].data_ptr(), _ptr(pci), _ptr(pbm_c), block_m, block_n, S,
                                  o_frp.data_ptr(), o_fci.data_ptr(), o_prp.data_ptr(), o_pci.data_ptr(),
                                  o_lrp.data_ptr(), o_lci.data_ptr(), o_bits.data_ptr(), counts.data_ptr(),
                                  tiles, tiles, tiles, ws.data_ptr(), ws.numel(), _stream(dev)), "stof_retile_lut")
        per_sample.append((o_frp, o_fci, o_prp, o_pci, o_lrp, o_lci, o_bits, counts))
    if lrp.dim() == 1:
        # one shared LUT: the lists stay at full capacity (entries past the last row pointer unused), nothing is read back
        o_frp, o_fci, o_prp, o_pci, o_lrp, o_lci, o_bits, _ = per_sample[0]
    else:
        # per-sample: exact lengths are needed to concatenate (one read of the counts per sample), row pointers become absolute
        fo = po = lo = 0
        parts = {k: [] for k in ("frp", "fci", "prp", "pci", "lrp", "lci", "bits")}
        for (a, bq, c, d, e, f, g, counts) in per_sample:
            n_full, n_part64, n_load, overflow = counts.tolist()
            assert not overflow
            parts["frp"].append(a + fo); parts["fci"].append(bq[:n_full])
            parts["prp"].append(c + po); parts["pci"].append(d[:n_part64])
            parts["lrp"].append(e + lo); parts["lci"].append(f[:n_load]); parts["bits"].append(g[:n_part64])
            fo += n_full; po += n_part64; lo += n_load
        st = lambda k: torch.stack(parts[k], 0).contiguous()
        ct = lambda k: torch.cat(parts[k], 0).contiguous()
        o_frp, o_fci, o_prp, o_pci, o_lrp, o_lci, o_bits = st("frp"), ct("fci"), st("prp"), ct("pci"), st("lrp"), ct("lci"), ct("bits")
    # The attention kernel reads bit rows, not additive blocks: a one-block placeholder carries them
    # (as masks.build_lut_device does), and the lists are in order by construction.
    o_pbm = torch.ones(1, 64, 64, dtype=torch.float16, device=dev)
    setattr(o_pbm, _BITS_ATTR, (_content_key(o_pbm), o_bits))
    setattr(o_pbm, _DEVICE_BUILT_ATTR, True)
    setattr(o_lci, _LUT_OK_ATTR, tuple(_content_key(t) for t in (o_lci, o_pci, o_lrp, o_prp)))
    setattr(o_lci, _DEVICE_BUILT_ATTR, True)
    lut64 = (o_frp, o_fci, o_prp, o_pci, o_pbm, o_lrp, o_lci)
    try:
        setattr(lci, _LUT64_ATTR, (key, lut64))
    except AttributeError:
        pass
    return lut64


_LUT_READY_ATTR = "_stof_lut_ready"


def _prepared_lut(lut, B, S, block_m, block_n, dev):
    """Validate a LUT and turn it into the seven pointers ``stof_block_attn_fwd`` takes plus the
    per-sample row-pointer stride.  The work (dtype / device / shape / ordering checks, bit
    packing of the partial blocks, re-tiling to 64 x 64) is done once per LUT: the result is
    kept on the LOAD column tensor, keyed by the identity and content version of all seven
    tensors, the problem size and the device, and it holds the tensors it points into."""
    a, b, c, d, e, f, lci = lut
    # (identity, storage address and content version of the seven tensors, spelled out: this runs on every call)
    key = (B, S, block_m, block_n, dev,
           id(a), a.data_ptr(), a._version, id(b), b.data_ptr(), b._version, id(c), c.data_ptr(), c._version,
           id(d), d.data_ptr(), d._version, id(e), e.data_ptr(), e._version, id(f), f.data_ptr(), f._version,
           id(lci), lci.data_ptr(), lci._version)
    cached = getattr(lci, _LUT_READY_ATTR, None)
    if cached is not None and cached[0] == key:
        return cached[1], cached[2], cached[5]
    frp, fci, prp, pci, pbm, lrp, lci = lut
    frp = _check_i32("full_row_ptr", frp, dev); fci = _check_i32("full_col_idx", fci, dev)
    prp = _check_i32("part_row_ptr", prp, dev); pci = _check_i32("part_col_idx", pci, dev)
    lrp = _check_i32("load_row_ptr", lrp, dev); lci_c = _check_i32("load_col_idx", lci, dev)
    _require(pbm.dtype == torch.float16 and pbm.device == dev, "part_block_mask must be fp16 on q's device")
    _require(S % block_m == 0 and S % block_n == 0, f"seq_len {S} not divisible by block {block_m}x{block_n}")
    nq = S // block_m
    if lrp.dim() == 2:
        _require(lrp.shape == (B, nq + 1) and frp.shape == lrp.shape and prp.shape == lrp.shape,
                 f"per-sample row pointers must be [{B}, {nq + 1}]")
        lut_bs = nq + 1
    else:
        _require(lrp.numel() == nq + 1 and frp.numel() == nq + 1 and prp.numel() == nq + 1,
                 f"row pointers must have {nq + 1} entries for seq_len {S}, block_m {block_m}")
        lut_bs = 0
    _check_lut_order(lrp, lci_c, prp, pci, S // block_n)
    if (block_m, block_n) != (64, 64):
        _require(S % 64 == 0, f"seq_len {S} must be a multiple of 64")
        frp, fci, prp, pci, pbm, lrp, lci_c = _lut_at_64((frp, fci, prp, pci, pbm, lrp, lci_c), S, block_m, block_n)
        lut_bs = S // 64 + 1 if lrp.dim() == 2 else 0
    bits = _packed_partial_bits(pbm)
    keep = (frp, fci, prp, pci, bits, lrp, lci_c)
    ptrs = tuple(_ptr(t) for t in keep)
    plans = {}   # rows per workgroup -> plan tensor (see _plan), filled on first use
    try:
        setattr(lci, _LUT_READY_ATTR, (key, ptrs, lut_bs, keep, tuple(lut), plans))   # holds what the key and the pointers refer to
    except AttributeError:
        pass
    return ptrs, lut_bs, plans


def _plan(plans, lut_ptrs, lut_bs, B, H, S, form, dev):
    """The precomputed walk of this LUT for the launch form the library will take (built by one
    small launch the first time a LUT meets that form, then kept with the LUT's other prepared
    data).  Returns (pointer, bytes, rows per workgroup) or (None, 0, 0) where no plan applies."""
    hit = plans.get((B, H, S, form))
    if hit is not None:
        return hit
    lib = _lib.lib()
    rows = lib.stof_attn_plan_rows(B, H, S, form)
    triple = (None, 0, 0)
    if rows > 0:
        plan = plans.get(rows)
        if plan is None:
            batches = B if lut_bs else 1
            nbytes = lib.stof_attn_plan_bytes(S, rows, batches)
            plan = False
            if nbytes > 0:
                plan = torch.empty(nbytes // 8, dtype=torch.int64, device=dev)
                check(lib.stof_attn_plan_build(lut_ptrs[2], lut_ptrs[3], lut_ptrs[5], lut_ptrs[6], S, lut_bs, batches, rows,
                                               plan.data_ptr(), nbytes, _stream(dev)), "stof_attn_plan_build")
            plans[rows] = plan
        if plan is not False:
            triple = (plan.data_ptr(), plan.numel() * 8, rows)
    plans[(B, H, S, form)] = triple
    return triple


def _check_i32(name, t, device):
    _require(t.dtype == torch.int32, f"{name} must be int32, got {t.dtype}")
    _require(t.device == device, f"{name} is on {t.device}, expected {device}")
    return t.contiguous()


def block_attn(q, k, v, lut, block_m=64, block_n=64, out=None, out_layout="bhsd", softmax_scale=None,
               launch_form=None, revalidate=False, use_plan=True, _bind=None):
    """Block-masked attention.  q, k, v: fp16 (or, all three, bfloat16) views ``[B,H,S,D]`` with
    unit stride in D (any other strides).  ``lut`` = (full_row_ptr, full_col_idx, part_row_ptr, part_col_idx,
    part_block_mask, load_row_ptr, load_col_idx) as returned by ``get_sparse_storage`` (the
    leading ``nnz`` dropped) or by ``get_sparse_storage_batched`` (2-D row pointers: one LUT
    per sample).  Returns ``out``: ``[B,H,S,D]`` (``out_layout='bhsd'``) or ``[B,S,H*D]``
    (``'bshd'``); ``out`` may be ``q`` itself.

    ``launch_form``: ``None`` / ``"default"`` (this module's default, automatic by grid size
    unless ``set_attention_launch_form`` changed it), ``"auto"``, ``"two_rows"`` or ``"key_split"`` - the
    per-call counterpart of the reference's ``num_warps``.  ``use_plan=False`` makes the kernel
    read the LUT itself instead of the walk laid out once per LUT (same result bit for bit; the
    plan saves the dependent LUT reads at the start of every workgroup).  ``revalidate=True`` discards what
    is cached for this LUT (validation, packed bit rows, re-tiling) and prepares it again: for
    LUT buffers rewritten behind PyTorch's back, which the caches cannot see.
    """
    if not q.is_cuda:
        raise StofError("q must be a CUDA tensor (this path has no CPU implementation)")
    dev = q.device
    dt = _DTYPES.get(q.dtype)
    if dt is None:
        raise StofError(f"q must be float16 or bfloat16, got {q.dtype}")
    qs, ks, vs = q.stride(), k.stride(), v.stride()
    for name, t, st in (("q", q, qs), ("k", k, ks), ("v", v, vs)):
        if t.dtype != q.dtype:
            raise StofError(f"{name} must be {q.dtype} like q, got {t.dtype}")
        if len(st) != 4 or st[3] != 1:
            raise StofError(f"{name} must be [B,H,S,D] with contiguous D")
        if t is not q and t.device != dev:
            raise StofError(f"{name} is on a different device than q")
    shape = q.shape
    if k.shape != shape or v.shape != shape:
        raise StofError("q, k, v must have the same shape")
    B, H, S, D = shape
    if out is None:
        out = torch.empty((B, H, S, D) if out_layout == "bhsd" else (B, S, H * D), dtype=q.dtype, device=dev)
    os_ = out.stride()
    if out_layout == "bhsd":
        if out.shape != shape or os_[3] != 1:
            raise StofError("out must be [B,H,S,D] with contiguous D")
        ostr = _lib.i64x3(os_[0], os_[1], os_[2])
    elif out_layout == "bshd":
        if out.shape != (B, S, H * D) or os_[2] != 1:
            raise StofError("out must be [B,S,H*D] with contiguous last dim")
        ostr = _lib.i64x3(os_[0], D, os_[1])
    else:
        raise StofError(f"unknown out_layout {out_layout!r}")
    if out.dtype != q.dtype or out.device != dev:
        raise StofError("out must have q's dtype and device")
    if _bind is None:
        return _attn_launch(q.data_ptr(), k.data_ptr(), v.data_ptr(), out, _lib.i64x3(qs[0], qs[1], qs[2]),
                            _lib.i64x3(ks[0], ks[1], ks[2]), _lib.i64x3(vs[0], vs[1], vs[2]), ostr, B, H, S, D, dt, dev,
                            lut, block_m, block_n, softmax_scale, launch_form, revalidate, use_plan)
    # BoundAttention: the arguments are kept, and the first launch happens with them
    _bind._args = _attn_args(q.data_ptr(), k.data_ptr(), v.data_ptr(), out, _lib.i64x3(qs[0], qs[1], qs[2]),
                             _lib.i64x3(ks[0], ks[1], ks[2]), _lib.i64x3(vs[0], vs[1], vs[2]), ostr, B, H, S, D, dt, dev,
                             lut, block_m, block_n, softmax_scale, launch_form, revalidate, use_plan)
    check(_lib.lib().stof_block_attn_fwd_planned(*_bind._args, _stream(dev)), "stof_block_attn_fwd")
    return out


def _attn_args(qp, kp, vp, out, qstr, kstr, vstr, ostr, B, H, S, D, dt, dev, lut, block_m, block_n,
               softmax_scale, launch_form, revalidate, use_plan):
    """The LUT side of an attention call (prepared data, plan): every argument of
    stof_block_attn_fwd_planned but the stream.  q, k, v arrive as validated device addresses with
    their (batch, head, row) element strides."""
    form = _form(launch_form)
    if revalidate:
        _drop_caches(lut)
    lut_ptrs, lut_bs, plans = _prepared_lut(lut, B, S, block_m, block_n, dev)
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    plan_ptr, plan_bytes, plan_rows = _plan(plans, lut_ptrs, lut_bs, B, H, S, form, dev) if use_plan else (None, 0, 0)
    return (qp, kp, vp, out.data_ptr(), *lut_ptrs, 64, 64, scale, qstr, kstr, vstr, ostr,
            B, S, H, D, dt, lut_bs, form, plan_ptr, plan_bytes, plan_rows)


def _attn_launch(qp, kp, vp, out, qstr, kstr, vstr, ostr, B, H, S, D, dt, dev, lut, block_m, block_n,
                 softmax_scale, launch_form, revalidate, use_plan):
    """The LUT side of an attention call and the launch (as _attn_args, spelled out once more: this
    is the per-call path and a tuple built and taken apart again shows in its cost)."""
    form = _form(launch_form)
    if revalidate:
        _drop_caches(lut)
    lut_ptrs, lut_bs, plans = _prepared_lut(lut, B, S, block_m, block_n, dev)
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    plan_ptr, plan_bytes, plan_rows = _plan(plans, lut_ptrs, lut_bs, B, H, S, form, dev) if use_plan else (None, 0, 0)
    check(_lib.lib().stof_block_attn_fwd_planned(
        qp, kp, vp, out.data_ptr(), *lut_ptrs, 64, 64, scale, qstr, kstr, vstr, ostr,
        B, S, H, D, dt, lut_bs, form, plan_ptr, plan_bytes, plan_rows, _stream(dev)), "stof_block_attn_fwd")
    return out


class BoundAttention:
    """``block_attn`` on fixed buffers with everything that does not change between calls resolved
    once: a serving loop that keeps q, k, v and the output in place (the way a captured graph does,
    for callers that cannot capture one) then pays the binding and the launch per call and none of
    the per-call validation, stride extraction and LUT look-up.

        run = BoundAttention(q, k, v, lut, out=out)      # validates, prepares the LUT, lays out the walk
        ...                                              # new contents written INTO q, k, v
        run()                                            # one launch on the current stream; returns out

    The addresses, shapes and strides of the four tensors and the LUT's prepared form are taken at
    construction and kept alive by this object.  Writing new values into the tensors is what it is
    for; re-allocating or resizing them, or changing the LUT, needs a new BoundAttention."""

    def __init__(self, q, k, v, lut, block_m=64, block_n=64, out=None, out_layout="bhsd", softmax_scale=None,
                 launch_form=None, use_plan=True):
        self._args = None
        self.out = block_attn(q, k, v, lut, block_m, block_n, out, out_layout, softmax_scale, launch_form,
                              use_plan=use_plan, _bind=self)
        self._keep = (q, k, v, lut, getattr(lut[6], _LUT_READY_ATTR, None))   # what the addresses point into
        self._dev = q.device
        self._fn = _lib.lib().stof_block_attn_fwd_planned

    def __call__(self):
        check(self._fn(*self._args, _stream(self._dev)), "stof_block_attn_fwd")
        return self.out


def block_attn_packed_qkv(qkv, n_heads, lut, block_m=64, block_n=64, out=None, softmax_scale=None,
                          launch_form=None, use_plan=True):
    """``block_attn`` on the packed projection ``qkv`` [B, S, 3*H*D] (q, k, v side by side in the
    last dim, each as H heads of D channels - what one QKV GEMM writes), result ``[B, S, H*D]``.
    The same launch as ``block_attn`` on the three strided views; this entry spares the nine
    view / permute operations that forming them costs on the host."""
    if not qkv.is_cuda:
        raise StofError("qkv must be a CUDA tensor (this path has no CPU implementation)")
    dt = _DTYPES.get(qkv.dtype)
    if dt is None:
        raise StofError(f"qkv must be float16 or bfloat16, got {qkv.dtype}")
    if qkv.dim() != 3 or qkv.stride(2) != 1 or qkv.shape[2] % (3 * n_heads) != 0:
        raise StofError("qkv must be [B, S, 3*H*D] with a contiguous last dim")
    B, S, D3 = qkv.shape
    Dm = D3 // 3
    D = Dm // n_heads
    dev = qkv.device
    if out is None:
        out = torch.empty((B, S, Dm), dtype=qkv.dtype, device=dev)
    elif out.shape != (B, S, Dm) or out.stride(2) != 1 or out.dtype != qkv.dtype or out.device != dev:
        raise StofError("out must be [B,S,H*D] with contiguous last dim, of qkv's dtype and device")
    sb, ss, _ = qkv.stride()
    st = _lib.i64x3(sb, D, ss)
    base = qkv.data_ptr()
    esz = 2
    return _attn_launch(base, base + Dm * esz, base + 2 * Dm * esz, out, st, st, st, _lib.i64x3(out.stride(0), D, out.stride(1)),
                        B, n_heads, S, D, dt, dev, lut, block_m, block_n, softmax_scale, launch_form, False, use_plan)


class Block_Attn_Mask(Function):
    """src/ops/package_op.py:50-68: the result is written into ``q`` and ``q`` is returned.
    A non-contiguous ``q`` also receives the result (the reference silently returns it
    unchanged in that case)."""

    @staticmethod
    def forward(ctx, q, k, v,
                full_row_ptr, full_col_idx,
                part_row_ptr, part_col_idx, part_block_mask,
                load_row_ptr, load_col_idx,
                BLOCK_M, BLOCK_N, num_warps):
        lut = (full_row_ptr, full_col_idx, part_row_ptr, part_col_idx, part_block_mask,
               load_row_ptr, load_col_idx)
        if k.stride(-1) != 1:
            k = k.contiguous()
        if v.stride(-1) != 1:
            v = v.contiguous()
        if q.stride(-1) == 1:
            block_attn(q, k, v, lut, BLOCK_M, BLOCK_N, out=q)
        else:
            q.copy_(block_attn(q.contiguous(), k, v, lut, BLOCK_M, BLOCK_N))
        ctx.mark_non_differentiable(q)
        return q


def _rowwise(kind, q, k, v, is_causal, bandwidth, row_mask, launch_form=None):
    _require(q.is_cuda, "q must be a CUDA tensor (this path has no CPU implementation)")
    _require(q.dtype in _DTYPES, f"q must be float16 or bfloat16, got {q.dtype}")
    for name, t in (("k", k), ("v", v)):
        _require(t.dtype == q.dtype, f"{name} must be {q.dtype} like q, got {t.dtype}")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    B, H, S, D = q.shape
    result = torch.zeros((B, S, H * D), device=q.device, dtype=q.dtype)
    bits = None
    if kind == 2:
        _require(row_mask.shape[-2:] == (S, S), f"row_mask must be [{S},{S}]")
        cached = getattr(row_mask, _BITS_ATTR, None)
        if cached is not None and cached[0] == _content_key(row_mask):
            bits = cached[1]
        else:
            bits = pack_mask_bits(row_mask.to(torch.float16).reshape(S, S), additive=False)
            try:
                setattr(row_mask, _BITS_ATTR, (_content_key(row_mask), bits))
            except AttributeError:
                pass
    check(_lib.lib().stof_rowwise_attn_fwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), result.data_ptr(),
        kind, 1 if is_causal else 0, int(bandwidth), _ptr(bits),
        B, S, H, D, _DTYPES[q.dtype], _form(launch_form), _stream(q.device)), "stof_rowwise_attn_fwd")
    return result


def rowwise_attn(kind, q, k, v, is_causal=False, bandwidth=0, row_mask=None, launch_form=None):
    """Functional form of the three row-wise operators with the launch form as an argument:
    ``kind`` "full" | "sliding" | "mask"; returns ``[B, S, H*D]``."""
    kinds = {"full": 0, "sliding": 1, "mask": 2}
    _require(kind in kinds, f"kind must be one of {sorted(kinds)}, got {kind!r}")
    return _rowwise(kinds[kind], q, k, v, is_causal, bandwidth, row_mask, launch_form)


class RowWise_Attn_Full(Function):
    """src/ops/package_op.py:11-22."""

    @staticmethod
    def forward(ctx, q, k, v, is_causal=False):
        result = _rowwise(0, q, k, v, is_causal, 0, None)
        ctx.mark_non_differentiable(result)
        return result


class RowWise_Attn_Sliding(Function):
    """src/ops/package_op.py:24-35."""

    @staticmethod
    def forward(ctx, q, k, v, is_causal, bandwidth):
        result = _rowwise(1, q, k, v, is_causal, bandwidth, None)
        ctx.mark_non_differentiable(result)
        return result


class RowWise_Attn_Mask(Function):
    """src/ops/package_op.py:37-48."""

    @staticmethod
    def forward(ctx, q, k, v, is_causal, row_mask):
        result = _rowwise(2, q, k, v, is_causal, 0, row_mask)
        ctx.mark_non_differentiable(result)
        return result


rowwise_attn_full_op = RowWise_Attn_Full.apply
rowwise_attn_sliding_op = RowWise_Attn_Sliding.apply
rowwise_attn_mask_op = RowWise_Attn_Mask.apply
block_attn_mask_op = Block_Attn_Mask.apply
