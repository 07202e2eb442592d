"""LUTs built with other block sizes (the reference's BLOCK_M / BLOCK_N of 16 .. 128,
src/ops/src/block_attn_mask_cuda.cu:6064-6322) re-tiled to 64 x 64 on the device: the re-tiled
lists and bit rows against the oracle's get_sparse_storage(mask, 64, 64) (bit for bit), attention
through them against the oracle (2e-3 + 1e-2 |want|), shared and per-sample LUTs, and the
``revalidate`` path of LUTs the library built on the device."""
import numpy as np
import pytest
import torch

from oracle import attention as oa
from oracle import masks as om
from stof import configs, masks as pm
from stof._cache import BITS_ATTR
from stof.ops import _lut_at_64, block_attn, block_attn_mask_op

pytestmark = pytest.mark.gpu
BLOCKS = [(16, 16), (32, 32), (128, 128), (32, 64), (64, 16), (128, 32), (16, 128)]


def _mask(S, seed):
    g = torch.Generator().manual_seed(seed)
    mask = configs.mask_c1(S).float()
    mask[200:330, 350:480] = (torch.rand(130, 130, generator=g) < 0.5).float()   # ragged patch of partial tiles
    mask[384:448, 0:64] = 1.0                                                     # a full 64 x 64 tile made of smaller full blocks
    return mask


def _close(got, want, what):
    err = (got.float().cpu() - want).abs()
    assert not bool((err > 2e-3 + 1e-2 * want.abs()).any()), f"{what}: max abs err {float(err.max()):.3e}"


def _oracle_lut64(mask2d):
    """(frp, fci, prp, pci, bit rows, lrp, lci) of the oracle at 64 x 64, bit rows packed on the host."""
    _, frp, fci, prp, pci, pbm, lrp, lci = om.get_sparse_storage(mask2d[None].numpy(), 64, 64)
    n_part = int(prp[-1])
    keep = (np.asarray(pbm[:n_part], dtype=np.float32) == 0)                      # [n,64,64] allowed
    bits = (keep.astype(np.uint64) << np.arange(64, dtype=np.uint64)[None, None, :]).sum(-1).astype(np.uint64)
    return [np.asarray(t) for t in (frp, fci, prp, pci)] + [bits] + [np.asarray(lrp), np.asarray(lci)]


@pytest.mark.parametrize("bm,bn", BLOCKS)
def test_retiled_lut_equals_the_oracle_at_64(bm, bn):
    S = 512
    mask = _mask(S, bm * 1000 + bn)
    lut = pm.get_sparse_storage(mask[None].cuda(), bm, bn)[1:]
    got = _lut_at_64(lut, S, bm, bn)
    want = _oracle_lut64(mask)
    n_full, n_part, n_load = int(want[0][-1]), int(want[2][-1]), int(want[5][-1])
    for name, g, w, n in (("full_row_ptr", got[0], want[0], None), ("full_col_idx", got[1], want[1], n_full),
                          ("part_row_ptr", got[2], want[2], None), ("part_col_idx", got[3], want[3], n_part),
                          ("load_row_ptr", got[5], want[5], None), ("load_col_idx", got[6], want[6], n_load)):
        g = g.cpu().numpy() if n is None else g.cpu().numpy()[:n]
        assert np.array_equal(g, np.asarray(w, dtype=g.dtype)), f"{name} at {bm}x{bn}"
    bits = getattr(got[4], BITS_ATTR)[1].cpu().numpy().view(np.uint64)[:n_part]
    assert np.array_equal(bits, want[4]), f"bit rows at {bm}x{bn}"


@pytest.mark.parametrize("bm,bn", BLOCKS)
def test_attention_through_a_retiled_lut(bm, bn):
    S = 512
    mask = _mask(S, bm * 1000 + bn)
    q, k, v = configs.qkv(configs.AttnConfig("t", 2, 3, S), seed=11, device="cuda")
    want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask.bool())
    lut = pm.get_sparse_storage(mask[None].cuda(), bm, bn)
    _close(block_attn(q, k, v, lut[1:], bm, bn), want, f"block {bm}x{bn}")
    _close(block_attn_mask_op(q.clone(), k, v, *lut[1:], bm, bn, 4), want, f"op, block {bm}x{bn}")


@pytest.mark.parametrize("bm,bn", [(16, 16), (32, 64), (128, 128), (128, 32)])
def test_per_sample_lut_at_other_block_sizes(bm, bn):
    """Key-padding x window masks, one LUT per sample, built at bm x bn and re-tiled sample by sample."""
    B, H, S = 3, 2, 512
    lens = [512, 333, 150]
    idx = torch.arange(S)
    masks = torch.stack([((idx[None, :] < L) & ((idx[:, None] - idx[None, :]).abs() <= 180)) for L in lens]).float()
    lut = pm.get_sparse_storage_batched(masks.cuda(), bm, bn)[1:]
    q, k, v = configs.qkv(configs.AttnConfig("p", B, H, S), seed=5, device="cuda")
    got = block_attn(q, k, v, lut, bm, bn)
    lut64 = pm.get_sparse_storage_batched(masks.cuda(), 64, 64)[1:]
    assert torch.equal(got, block_attn(q, k, v, lut64)), "re-tiled per-sample LUT gives other bits than the 64 x 64 LUT"
    for b, L in enumerate(lens):
        want = oa.dense_masked_attention(q[b:b + 1].cpu().float(), k[b:b + 1].cpu().float(), v[b:b + 1].cpu().float(), masks[b].bool())
        _close(got[b:b + 1, :, :L], want[:, :, :L], f"sample {b} at {bm}x{bn}")


def test_revalidate_on_device_built_luts():
    """revalidate=True on a LUT whose bit rows exist only on the device (build_lut_device, a
    re-tiled LUT): the library's own attachments stay, the result is unchanged."""
    S = 512
    mask = _mask(S, 3)
    q, k, v = configs.qkv(configs.AttnConfig("t", 1, 4, S), seed=2, device="cuda")
    want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask.bool())
    lut = pm.build_lut_device(mask[None].cuda().half())
    a = block_attn(q, k, v, lut)
    b = block_attn(q, k, v, lut, revalidate=True)
    assert torch.equal(a, b)
    _close(b, want, "device-built LUT, revalidate")
    lut32 = pm.get_sparse_storage(mask[None].cuda(), 32, 32)[1:]
    c = block_attn(q, k, v, lut32, 32, 32)
    d = block_attn(q, k, v, lut32, 32, 32, revalidate=True)
    assert torch.equal(c, d)
    _close(d, want, "re-tiled LUT, revalidate")
