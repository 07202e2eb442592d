"""The mask -> block LUT kernels (stof_build_lut, stof_lut_additive_blocks) on the GPU, bit for
bit against the CPU oracle's restatement of get_sparse_storage (src/util/masks.py:125-184)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import attention as oa
from oracle import masks as om
from stof import _lib, configs, masks as pm
from stof._cache import BITS_ATTR
from stof.ops import block_attn

pytestmark = pytest.mark.gpu


def _same_lut(got, want, bm, bn, what):
    """got: the product's 8-tuple (device tensors); want: the oracle's (numpy)."""
    names = ["nnz", "full_row_ptr", "full_col_idx", "part_row_ptr", "part_col_idx", "part_block_mask", "load_row_ptr", "load_col_idx"]
    # (the non-zero count comes out of the classification pass; the figure is the reference's float32 arithmetic)
    assert np.float32(float(got[0])) == np.float32(float(want[0])), f"{what}: nnz {float(got[0])} vs {float(want[0])}"
    for i in (1, 2, 3, 4, 6, 7):
        g = got[i].cpu().numpy()
        assert g.dtype == np.int32 and g.shape == want[i].shape and np.array_equal(g, want[i]), f"{what}: {names[i]} differs"
    g = got[5].cpu().numpy()
    assert g.dtype == np.float16 and g.shape == want[5].shape, f"{what}: part_block_mask shape {g.shape} vs {want[5].shape}"
    assert np.array_equal(g.view(np.uint16), want[5].view(np.uint16)), f"{what}: part_block_mask bits differ"


def _bit_rows(additive):
    """[n,64,64] additive fp16 blocks -> uint64 [n,64] bit rows (bit j = key j allowed)."""
    keep = (additive.astype(np.float32) > -5000).astype(np.uint64)
    return (keep << np.arange(64, dtype=np.uint64)[None, None, :]).sum(-1)


@pytest.mark.parametrize("name", ["C1", "C2", "C4", "C5"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_baseline_masks_bit_identical_on_device(name, dtype):
    s = {"C1": 512, "C2": 1024, "C4": 4096, "C5": 2048}[name]
    mask = configs.ATTN_MASKS[name](s)
    dev_mask = mask.to(dtype)[None].cuda()
    got = pm.get_sparse_storage(dev_mask, 64, 64)
    want = om.get_sparse_storage(mask.float()[None].numpy(), 64, 64)
    _same_lut(got, want, 64, 64, f"{name} {dtype}")
    full, part = configs.BLOCK_COUNTS[name]
    assert int(got[1][-1]) == full and int(got[3][-1]) == part
    bits = getattr(got[5], BITS_ATTR, None)
    if part:
        assert bits is not None, "the kernel's bit rows were not handed to the attention operator"
        assert np.array_equal(bits[1].cpu().numpy().view(np.uint64), _bit_rows(want[5])), f"{name}: bit rows differ"


@pytest.mark.parametrize("bm,bn", [(64, 64), (32, 32), (16, 64), (128, 64), (64, 128), (16, 16), (128, 128)])
@pytest.mark.parametrize("seed", [0, 1])
def test_random_masks_and_block_sizes(bm, bn, seed):
    """Random tile classes (empty / full / sparse partial / dense partial / a single 0 or 1 in a
    corner), rows of one class only, for every supported block shape."""
    g = torch.Generator().manual_seed(100 + seed)
    S = 768 if max(bm, bn) > 64 else 384
    nq, nk = S // bm, S // bn
    kind = torch.randint(0, 5, (nq, nk), generator=g)
    kind[0, :] = 0; kind[1 % nq, :] = 1                     # an empty row of tiles, a full one
    mask = torch.zeros(S, S)
    for r in range(nq):
        for c in range(nk):
            t = mask[r * bm:(r + 1) * bm, c * bn:(c + 1) * bn]
            k = int(kind[r, c])
            if k == 1: t.fill_(1)
            elif k == 2: t.copy_((torch.rand(bm, bn, generator=g) < 0.1).float())
            elif k == 3: t.fill_(1); t[bm - 1, bn - 1] = 0
            elif k == 4: t[0, 0] = 1
    for dtype in (torch.float16, torch.float32):
        got = pm.get_sparse_storage(mask.to(dtype)[None].cuda(), bm, bn)
        want = om.get_sparse_storage(mask[None].numpy(), bm, bn)
        _same_lut(got, want, bm, bn, f"random {bm}x{bn} seed {seed} {dtype}")


def test_batch_zero_only_strided_rows_and_batched():
    """The LUT describes batch 0 (src/util/masks.py:147); rows at a pitch above S; per-sample LUTs."""
    g = torch.Generator().manual_seed(7)
    B, S = 3, 256
    mask = (torch.rand(B, S, S, generator=g) < 0.5).float()
    mask[:, :64, :128] = 1; mask[:, 64:128, :64] = 0
    got = pm.get_sparse_storage(mask.half().cuda(), 64, 64)
    _same_lut(got, om.get_sparse_storage(mask.numpy(), 64, 64), 64, 64, "batch 0")
    wide = torch.zeros(B, S, S + 64).half().cuda()
    wide[:, :, :S] = mask.half().cuda()
    got = pm.get_sparse_storage(wide[:, :, :S], 64, 64)               # a view: row pitch S + 64
    _same_lut(got, om.get_sparse_storage(mask.numpy(), 64, 64), 64, 64, "strided rows")
    gb = pm.get_sparse_storage_batched(mask.half().cuda(), 64, 64)
    cb = pm.get_sparse_storage_batched(mask, 64, 64)                  # the tensor-op path on the CPU
    for a, b in zip(gb[1:], cb[1:]):
        assert torch.equal(a.cpu(), b), "batched LUT differs between the GPU kernels and the tensor-op path"


def test_device_lut_feeds_attention_without_a_host_round_trip():
    cfg = configs.AttnConfig("t", 2, 4, 2048)
    mask = configs.mask_c5(cfg.seq)
    q, k, v = configs.qkv(cfg, seed=3, device="cuda")
    lut = pm.build_lut_device(mask.half()[None].cuda())
    got = block_attn(q, k, v, lut)
    want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask)
    err = (got.float().cpu() - want).abs()
    assert bool((err <= 2e-3 + 1e-2 * want.abs()).all()), f"max abs err {float(err.max()):.3e}"
    assert torch.equal(got, block_attn(q, k, v, pm.get_sparse_storage(mask.half()[None].cuda(), 64, 64)[1:]))


def test_capacity_too_small_is_reported_not_overrun():
    lib = _lib.lib()
    S = 256
    mask = torch.ones(S, S, dtype=torch.float16, device="cuda")
    mask[0, 0] = 0                                                     # 15 full tiles + 1 partial
    i32 = lambda n: torch.full((n,), -7, dtype=torch.int32, device="cuda")
    frp, prp, lrp = i32(5), i32(5), i32(5)
    fci, pci, lci = i32(16), i32(16), i32(16)
    counts = i32(4)
    ws = torch.empty(lib.stof_build_lut_workspace_bytes(S, 64, 64), dtype=torch.uint8, device="cuda")
    rc = lib.stof_build_lut(mask.data_ptr(), 2, S, S, 64, 64, frp.data_ptr(), fci.data_ptr(), prp.data_ptr(), pci.data_ptr(),
                            lrp.data_ptr(), lci.data_ptr(), None, counts.data_ptr(), 4, 16, 16, ws.data_ptr(), ws.numel(), None)
    assert rc == 0
    torch.cuda.synchronize()
    assert counts.tolist() == [15, 1, 16, 1]                           # full list truncated: flagged
    assert fci[4:].eq(-7).all() and lrp.tolist() == [0, 4, 8, 12, 16]  # nothing written past the capacity


def test_nnz_counts_every_batch_and_any_non_zero_value():
    """nnz is the count of non-zero elements of the WHOLE [B,S,S] tensor over S*S (src/util/masks.py:137):
    batch 0 counted by the kernels, the other batches by torch; values other than 0 / 1 count as non-zero."""
    S = 256
    g = torch.Generator().manual_seed(5)
    m = (torch.rand(3, S, S, generator=g) < 0.3).float()
    m[0, 5, 7] = 0.5; m[0, 9, 200] = 2.0
    for dtype in (torch.float16, torch.float32):
        got = pm.get_sparse_storage(m.to(dtype).cuda(), 32, 64)
        want = om.get_sparse_storage(m.numpy(), 32, 64)
        assert np.float32(float(got[0])) == np.float32(float(want[0])), (float(got[0]), float(want[0]))
        assert got[0].device.type == "cuda"


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_values_other_than_zero_and_one(dtype):
    """The classification is by value (a tile is FULL iff every element == 1, absent iff every element == 0)
    and the bit rows follow the additive rule (-10000 * (1 - x) in fp16 above -5000): -0.0, values around
    0.5 and 1, large, negative, infinite and NaN entries must come out as the oracle and the packed additive
    blocks have them; the non-zero count takes every value that is not +-0."""
    S = 256
    g = torch.Generator().manual_seed(17)
    m = (torch.rand(S, S, generator=g) < 0.5).float()
    m[:64, :64] = 1.0; m[:64, 64:128] = 0.0; m[64:128, :64] = -0.0        # a full, an empty and a minus-zero tile
    m[64:128, 64:128] = 1.0; m[70, 70] = 1.0 + 2.0 ** -10                   # all ones but one element just above
    m[128:192, 0:64] = 0.0; m[130, 3] = 2.0 ** -20                          # all zeros but one tiny element
    odd = [0.5, 0.5 + 2.0 ** -11, 0.5 - 2.0 ** -12, 0.25, 0.75, 2.0, -1.0, 60000.0, float("inf"), float("-inf"), float("nan"), -0.0, 1e-7]
    for i, val in enumerate(odd):
        m[200 + i, 130 + 3 * i] = val
    dev_mask = m.to(dtype)[None].cuda()
    got = pm.get_sparse_storage(dev_mask, 64, 64)
    with np.errstate(over="ignore"):   # (60000 and inf overflow the additive form on purpose)
        want = om.get_sparse_storage(m.to(dtype).float()[None].numpy(), 64, 64)     # (the oracle sees the values the device holds)
    for i in (1, 2, 3, 4, 6, 7):
        assert np.array_equal(got[i].cpu().numpy(), want[i]), f"list {i} differs"
    assert np.float32(float(got[0])) == np.float32(float(want[0]))
    pbm = got[5].cpu().numpy()
    both_nan = np.isnan(pbm) & np.isnan(want[5])          # (a NaN's sign and payload are not part of the contract)
    differ = (pbm.view(np.uint16) != want[5].view(np.uint16)) & ~both_nan
    assert not differ.any(), f"additive blocks differ at {np.argwhere(differ)[:5].tolist()}: {pbm[differ][:5]} vs {want[5][differ][:5]}"
    bits = getattr(got[5], BITS_ATTR, None)
    assert bits is not None
    assert np.array_equal(bits[1].cpu().numpy().view(np.uint64), _bit_rows(pbm)), "bit rows differ from the additive rule"
