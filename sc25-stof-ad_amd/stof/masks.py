"""Mask specification and the mask -> block-LUT compiler (host side, PyTorch).

Same call signatures and return values as the reference's ``src/util/masks.py``:
five dense-mask generators (``:10-122``) and ``get_sparse_storage`` (``:125-184``),
which classifies every (query block, key block) tile of ``Mask[0]`` as full,
partial or empty and returns three CSR-like int32 lists plus the additive fp16
blocks of the partial tiles.  Outputs are bit-identical to the reference's; the
implementation is not a loop translation: every generator is a closed-form index
predicate evaluated once on the mask's device, and the classifier is a single
blocked reduction, so the compile step costs a handful of tensor ops where the
reference runs (S/bm)*(S/bn) ``torch.all`` calls.

Extensions that the reference lacks (its LUT is shared by the whole batch):
``get_sparse_storage_batched`` builds one LUT per sample and concatenates them
with absolute offsets, so that B == 1 degenerates to the reference format.
"""
import random

import torch

from . import _lib
from ._cache import BITS_ATTR, DEVICE_BUILT_ATTR, LUT_OK_ATTR, content_key
from .ops import _stream

NEG_MASK = -10000.0


def _grid(seq_len, device):
    i = torch.arange(seq_len, device=device)[:, None]
    j = torch.arange(seq_len, device=device)[None, :]
    return i, j


def _finish(attr_mask, allowed, is_causal):
    """Broadcast one [S,S] bool pattern over the batch in attr_mask's dtype and
    apply the reference's causal trim, which reaches the LAST batch entry only
    (its loop variable is used after the loop: src/util/masks.py:28-30)."""
    out = allowed.to(attr_mask.dtype).unsqueeze(0).repeat(attr_mask.shape[0], 1, 1)
    if is_causal:
        s = attr_mask.shape[1]
        i, j = _grid(s, attr_mask.device)
        out[-1] = out[-1] * (j <= i).to(attr_mask.dtype)
    return out


def generate_causal_mask(attr_mask):
    """src/util/masks.py:10-14: lower-triangular ones; float32 on the CPU whatever
    attr_mask's dtype and device are, exactly as the reference returns it."""
    seq_len = attr_mask.shape[1]
    tri = torch.tril(torch.ones(seq_len, seq_len))
    return tri.unsqueeze(0).repeat(attr_mask.shape[0], 1, 1)


def generate_sliding_mask(attr_mask, bandwidth=1, is_cauasl=False):
    """src/util/masks.py:17-32: 1 where |i-j| <= bandwidth."""
    i, j = _grid(attr_mask.shape[1], attr_mask.device)
    return _finish(attr_mask, (i - j).abs() <= bandwidth, is_cauasl)


def generate_dilated_mask(attr_mask, bandwidth=1, dilation_rate=1, is_cauasl=False):
    """src/util/masks.py:35-52: 1 at columns i-bw-d + t*(d+1), t >= 0, that lie in
    [0, min(S, i+bw+d+1))."""
    s = attr_mask.shape[1]
    i, j = _grid(s, attr_mask.device)
    w = bandwidth + dilation_rate
    off = j - (i - w)
    allowed = (off >= 0) & (off % (dilation_rate + 1) == 0) & (j < torch.clamp(i + w + 1, max=s))
    return _finish(attr_mask, allowed, is_cauasl)


def generate_longformer_mask(attr_mask, globalwidth=1, bandwidth=1, is_cauasl=False):
    """src/util/masks.py:55-81: global rows/columns [0,g) and [S/2, S/2+g) plus the band."""
    s = attr_mask.shape[1]
    i, j = _grid(s, attr_mask.device)
    lo, hi = int(s / 2), int(s / 2 + globalwidth)
    glob = (i < globalwidth) | (j < globalwidth) | ((i >= lo) & (i < hi)) | ((j >= lo) & (j < hi))
    return _finish(attr_mask, glob | ((i - j).abs() <= bandwidth), is_cauasl)


def generate_bigbird_mask(attr_mask, globalwidth=1, bandwidth=1, fill_rate=0.2, is_cauasl=False):
    """src/util/masks.py:86-122: global + band + random points.

    The random points come from the stdlib generator seeded with 0 and consumed in
    the reference's order (per batch, per 32-row block: one ``choice`` for the
    column block, then ``randint(0,32)`` for x and y of each of
    ``int(1024*fill_rate)`` points), so the mask is reproducible bit for bit.
    """
    b, s = attr_mask.shape[0], attr_mask.shape[1]
    i, j = _grid(s, attr_mask.device)
    base = (i < globalwidth) | (j < globalwidth) | ((i - j).abs() <= bandwidth)
    out = base.to(attr_mask.dtype).unsqueeze(0).repeat(b, 1, 1)
    npts = int(1024 * fill_rate)
    random.seed(0)
    nblk = int(s / 32)
    bb, xx, yy = [], [], []
    for batch in range(b):
        for blk in range(nblk - 1):
            sx = blk * 32
            if blk == 0:
                sy = sx + 32 * random.choice([1, 0])
            elif blk == nblk - 2:
                sy = sx + 32 * random.choice([-1, 0])
            else:
                sy = sx + 32 * random.choice([-1, 0, 1])
            for _ in range(npts):
                xx.append(sx + random.randint(0, 32))
                yy.append(sy + random.randint(0, 32))
                bb.append(batch)
    if bb:
        dev = attr_mask.device
        out[torch.tensor(bb, device=dev), torch.tensor(xx, device=dev), torch.tensor(yy, device=dev)] = 1
    if is_cauasl:
        out[-1] = out[-1] * (j <= i).to(attr_mask.dtype)
    return out


def _classify(m2d, bm, bn):
    """[S,S] -> (blocks [nQ,nK,bm,bn], full [nQ,nK] bool, part [nQ,nK] bool)."""
    n = m2d.shape[-1]
    if m2d.shape[-2] != n or n % bm or n % bn:
        raise ValueError(f"mask must be square with seq_len divisible by the block sizes; "
                         f"got {tuple(m2d.shape)} for blocks {bm}x{bn}")
    blocks = m2d.reshape(n // bm, bm, n // bn, bn).permute(0, 2, 1, 3)
    full = (blocks == 1).all(-1).all(-1)
    empty = (blocks == 0).all(-1).all(-1)
    return blocks, full, ~full & ~empty


def _csr(flag):
    """[nQ,nK] bool -> (row_ptr int32 [nQ+1], col_idx int32 [nnz]) in row-major order."""
    counts = flag.sum(1)
    row_ptr = torch.zeros(flag.shape[0] + 1, dtype=torch.int64, device=flag.device)
    row_ptr[1:] = torch.cumsum(counts, 0)
    col_idx = flag.nonzero()[:, 1]
    return row_ptr.to(torch.int32), col_idx.to(torch.int32)


_DEVICE_BLOCKS = (16, 32, 64, 128)


def _device_path(Mask, bm, bn):
    """The GPU kernels take fp16 / fp32 masks with 16-byte aligned rows and block sizes of 16..128."""
    n = Mask.shape[-1]
    return (Mask.is_cuda and Mask.dtype in (torch.float16, torch.float32) and bm in _DEVICE_BLOCKS and bn in _DEVICE_BLOCKS
            and Mask.dim() == 3 and Mask.shape[-2] == n and n % bm == 0 and n % bn == 0 and (n * Mask.element_size()) % 16 == 0)


def _build_on_device(m2d, bm, bn, want_bits):
    """One sample's mask [S,S] on the GPU -> (row pointers x3, column lists x3 at full capacity,
    bit rows or None, counts tensor).  No synchronisation: everything stays on the device."""
    if m2d.stride(1) != 1 or (m2d.stride(0) * m2d.element_size()) % 16 or m2d.data_ptr() % 16:
        m2d = m2d.contiguous()
    n = m2d.shape[-1]
    nq, nk = n // bm, n // bn
    tiles = nq * nk
    dev = m2d.device
    # one allocation for the six index arrays, cut up by one call
    idx = torch.empty(3 * (nq + 1) + 3 * tiles, dtype=torch.int32, device=dev)
    frp, prp, lrp, fci, pci, lci = idx.split((nq + 1, nq + 1, nq + 1, tiles, tiles, tiles))
    bits = torch.empty((tiles, 64), dtype=torch.int64, device=dev) if (want_bits and bm == 64 and bn == 64) else None
    lib = _lib.lib()
    # The workspace ends with the mask's non-zero count (int64), that count as the reference's percentage
    # (float32) and 4 spare bytes; the four list counts are placed right behind it, so that one device ->
    # host read of 32 bytes brings all of them.
    wbytes = lib.stof_build_lut_workspace_bytes(n, bm, bn)
    ws = torch.empty(wbytes + 16, dtype=torch.uint8, device=dev)
    counts = ws[wbytes - 16:].view(torch.int64)          # [nnz, nnz % as float32 | spare, n_full | n_part << 32, n_load | overflow << 32]
    _lib.check(lib.stof_build_lut(m2d.data_ptr(), m2d.element_size(), m2d.stride(0), n, bm, bn,
                                  frp.data_ptr(), fci.data_ptr(), prp.data_ptr(), pci.data_ptr(), lrp.data_ptr(), lci.data_ptr(),
                                  bits.data_ptr() if bits is not None else None, ws.data_ptr() + wbytes,
                                  tiles, tiles, tiles, ws.data_ptr(), wbytes, _stream(dev)), "stof_build_lut")
    return m2d, frp, fci, prp, pci, lrp, lci, bits, counts


def _read_counts(counts):
    """(non-zero elements, n_full, n_part, n_load, overflow) from the 32 bytes behind the workspace: one read."""
    nnz, _, a, b = counts.tolist()
    return nnz, a & 0xFFFFFFFF, (a >> 32) & 0xFFFFFFFF, b & 0xFFFFFFFF, (b >> 32) & 0xFFFFFFFF


def _get_sparse_storage_device(m2d, bm, bn):
    """The seven LUT tensors of one sample, exactly shaped, built by the GPU kernels (one
    device -> host read of the three list lengths)."""
    m2d, frp, fci, prp, pci, lrp, lci, bits, counts = _build_on_device(m2d, bm, bn, want_bits=True)
    nonzero, n_full, n_part, n_load, overflow = _read_counts(counts)
    assert not overflow
    n = m2d.shape[-1]
    fci, pci, lci = fci[:n_full], pci[:n_part], lci[:n_load]
    if n_part == 0:
        pbm = torch.ones(1, bm, bn, dtype=torch.float16, device=m2d.device)
    else:
        pbm = torch.empty(n_part, bm, bn, dtype=torch.float16, device=m2d.device)
        _lib.check(_lib.lib().stof_lut_additive_blocks(m2d.data_ptr(), m2d.element_size(), m2d.stride(0), n, bm, bn,
                                                       prp.data_ptr(), pci.data_ptr(), n_part, pbm.data_ptr(),
                                                       _stream(m2d.device)), "stof_lut_additive_blocks")
        if bits is not None:   # the attention operator finds the bit rows of these blocks already packed
            setattr(pbm, BITS_ATTR, (content_key(pbm), bits[:n_part]))
    return nonzero, counts, (frp, fci, prp, pci, pbm, lrp, lci)


def get_sparse_storage(Mask, block_size_m, block_size_n):
    """src/util/masks.py:125-184.  Mask [B,S,S] of 0/1 (any float dtype, any device).

    Returns ``(nnz, full_row_ptr, full_col_idx, part_row_ptr, part_col_idx,
    part_block_mask, load_row_ptr, load_col_idx)`` on Mask's device: ``nnz`` is the
    percentage of non-zeros of the WHOLE tensor over S*S (:137), the LUT describes
    batch 0 only (:147), partial tiles carry ``-10000 * (1 - block.half())`` (:160)
    and an LUT without partial tiles carries one dummy block of ones (:179-180).

    An fp16 / fp32 mask on the GPU is compiled by the library's kernels (one pass over the
    mask, stof_build_lut); anything else by the tensor operations below on the mask's device.
    Both give the same tensors bit for bit.
    """
    n = Mask.shape[-1]
    if _device_path(Mask, block_size_m, block_size_n):
        # the non-zero count of batch 0 comes out of the classification pass; further batches (which the
        # LUT ignores, but the reference's figure counts) are counted by torch
        nonzero, counts, lut = _get_sparse_storage_device(Mask[0], block_size_m, block_size_n)
        if Mask.shape[0] == 1:
            # the kernel has left the figure on the device in the reference's own arithmetic (a view of the
            # 32-byte counts block at the workspace's end: no host -> device copy for one number)
            return (counts.view(torch.float32)[2],) + lut
        nonzero += int(torch.count_nonzero(Mask[1:]))
        import numpy as np
        # (the reference's arithmetic: an int64 count / int * int in float32, src/util/masks.py:137)
        nnz = torch.tensor(float(np.float32(nonzero) / np.float32(n * n) * np.float32(100)), device=Mask.device)
        return (nnz,) + lut
    nnz = torch.count_nonzero(Mask) / (n * n) * 100
    blocks, full, part = _classify(Mask[0], block_size_m, block_size_n)
    full_row_ptr, full_col_idx = _csr(full)
    part_row_ptr, part_col_idx = _csr(part)
    load_row_ptr, load_col_idx = _csr(full | part)
    if int(part_row_ptr[-1]) == 0:
        part_block_mask = torch.ones(1, block_size_m, block_size_n, dtype=torch.float16, device=Mask.device)
    else:
        part_block_mask = (NEG_MASK * (1.0 - blocks[part].to(torch.float16))).contiguous()
    return (nnz, full_row_ptr, full_col_idx, part_row_ptr, part_col_idx,
            part_block_mask, load_row_ptr, load_col_idx)


def build_lut_device(Mask, block_size_m=64, block_size_n=64):
    """Mask [B,S,S] (fp16 / fp32, on the GPU) -> LUT of batch 0 without any device -> host
    synchronisation, for use with ``stof.ops.block_attn``: the same seven tensors as
    ``get_sparse_storage`` (without ``nnz``), except that the three column lists keep their
    full capacity (entries beyond the last row pointer are unused) and ``part_block_mask`` is a
    one-block placeholder that carries the partial tiles' packed bit rows, which is what the
    attention kernel reads.  64 x 64 blocks only."""
    if not _device_path(Mask, block_size_m, block_size_n) or (block_size_m, block_size_n) != (64, 64):
        raise ValueError("build_lut_device needs an fp16 / fp32 [B,S,S] mask on the GPU and 64 x 64 blocks")
    _, frp, fci, prp, pci, lrp, lci, bits, _ = _build_on_device(Mask[0], 64, 64, want_bits=True)
    pbm = torch.ones(1, 64, 64, dtype=torch.float16, device=Mask.device)
    setattr(pbm, BITS_ATTR, (content_key(pbm), bits))
    setattr(lci, LUT_OK_ATTR, tuple(content_key(t) for t in (lci, pci, lrp, prp)))   # in order by construction
    # (block_attn(..., revalidate=True) leaves these two attachments in place: there is nothing to derive them from again)
    setattr(pbm, DEVICE_BUILT_ATTR, True); setattr(lci, DEVICE_BUILT_ATTR, True)
    return frp, fci, prp, pci, pbm, lrp, lci


def get_sparse_storage_batched(Mask, block_size_m, block_size_n):
    """One LUT per sample.  Row pointers have shape [B, nQ+1] and hold ABSOLUTE
    offsets into the concatenated column lists / partial-block stack, so sample b's
    query block r owns entries ``row_ptr[b,r] .. row_ptr[b,r+1]``; with B == 1 the
    arrays equal get_sparse_storage's (row pointers gain a leading dim of 1).
    The reference has no counterpart: its kernel shares one LUT over the batch.
    """
    B, n = Mask.shape[0], Mask.shape[-1]
    nnz = torch.count_nonzero(Mask) / (n * n) * 100
    outs = {k: [] for k in ("frp", "fci", "prp", "pci", "pbm", "lrp", "lci")}
    fo = po = lo = 0
    on_device = _device_path(Mask, block_size_m, block_size_n)
    for b in range(B):
        if on_device:
            _, _, (frp, fci, prp, pci, pbm_b, lrp, lci) = _get_sparse_storage_device(Mask[b], block_size_m, block_size_n)
        else:
            blocks, full, part = _classify(Mask[b], block_size_m, block_size_n)
            frp, fci = _csr(full); prp, pci = _csr(part); lrp, lci = _csr(full | part)
            pbm_b = (NEG_MASK * (1.0 - blocks[part].to(torch.float16))) if pci.numel() else None
        outs["frp"].append(frp + fo); outs["fci"].append(fci)
        outs["prp"].append(prp + po); outs["pci"].append(pci)
        outs["lrp"].append(lrp + lo); outs["lci"].append(lci)
        if pci.numel():
            outs["pbm"].append(pbm_b)
        fo += fci.numel(); po += pci.numel(); lo += lci.numel()
    if po == 0:
        pbm = torch.ones(1, block_size_m, block_size_n, dtype=torch.float16, device=Mask.device)
    else:
        pbm = torch.cat(outs["pbm"], 0).contiguous()
    st = lambda k: torch.stack(outs[k], 0).contiguous()
    ct = lambda k: torch.cat(outs[k], 0).contiguous()
    return (nnz, st("frp"), ct("fci"), st("prp"), ct("pci"), pbm, st("lrp"), ct("lci"))


def expand_sparse_storage(lut, n, block_size_m, block_size_n):
    """LUT -> dense [n,n] float32 0/1 mask (full -> 1, partial -> additive block == 0).
    The inverse of get_sparse_storage on 0/1 masks; used to validate a LUT."""
    _, frp, fci, prp, pci, pbm, _, _ = lut
    nq, nk = n // block_size_m, n // block_size_n
    dev = frp.device
    out = torch.zeros(nq, nk, block_size_m, block_size_n, dtype=torch.float32, device=dev)
    rows_f = torch.repeat_interleave(torch.arange(nq, device=dev), (frp[1:] - frp[:-1]).long())
    out[rows_f, fci.long()] = 1
    if int(prp[-1]) > 0:
        rows_p = torch.repeat_interleave(torch.arange(nq, device=dev), (prp[1:] - prp[:-1]).long())
        out[rows_p, pci.long()] = (pbm.float() == 0).float()
    return out.permute(0, 2, 1, 3).reshape(n, n)
