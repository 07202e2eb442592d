"""Pins the attention oracle (oracle/attention.py): library routine (SDPA with a boolean
mask), float64 brute force, special cases and invariants.  No reference code is run."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oa
from oracle import masks as om
from stof import configs


def _qkv(b, h, s, d=64, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(b, h, s, d, generator=g).to(dtype) for _ in range(3))


def _bruteforce64(q, k, v, mask):
    """Element-by-element float64 evaluation of softmax(q.k/sqrt(d) over allowed j) v."""
    q, k, v = (t.double().numpy() for t in (q, k, v))
    B, H, S, D = q.shape
    out = np.zeros_like(q)
    for b in range(B):
        for h in range(H):
            for i in range(S):
                idx = [j for j in range(S) if mask[b, i, j]]
                if not idx:
                    continue
                sc = np.array([q[b, h, i] @ k[b, h, j] for j in idx]) / math.sqrt(D)
                w = np.exp(sc - sc.max()); w /= w.sum()
                out[b, h, i] = sum(wj * v[b, h, j] for wj, j in zip(w, idx))
    return out


def test_dense_vs_bruteforce_float64():
    q, k, v = _qkv(2, 2, 24, 8, seed=1)
    rng = np.random.default_rng(0)
    mask = (rng.random((2, 24, 24)) < 0.4)
    mask[0, 5] = False                       # a row without any allowed key -> zeros
    got = oa.dense_masked_attention(q, k, v, torch.from_numpy(mask), torch.float64).numpy()
    want = _bruteforce64(q, k, v, mask)
    assert np.abs(got - want).max() < 1e-12
    assert np.all(got[0, :, 5] == 0)


def test_dense_vs_sdpa_library():
    q, k, v = _qkv(2, 3, 128, 64, seed=2)
    mask = configs.mask_c1(128)[None].expand(2, -1, -1)
    got = oa.dense_masked_attention(q, k, v, mask)
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=mask[:, None])
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)


def test_torch_attn_std_matches_additive_definition():
    """the -10000 additive form equals hard masking for rows with an allowed key."""
    q, k, v = _qkv(1, 2, 64, 16, seed=3)
    mask = torch.tril(torch.ones(64, 64))[None]
    a = oa.torch_attn_std(q, k, v, mask)
    b = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert torch.allclose(a, b, atol=2e-6, rtol=1e-5)


def _lut(mask2d, bm=64, bn=64):
    return om.get_sparse_storage(mask2d.numpy().astype(np.float32)[None], bm, bn)


@pytest.mark.parametrize("name,s", [("C1", 512), ("C5", 256), ("C4", 512)])
def test_block_algorithm_equals_dense(name, s):
    mask = configs.ATTN_MASKS[name](s)
    q, k, v = _qkv(1, 2, s, 64, seed=4)
    got = oa.block_attn_mask(q.numpy(), k.numpy(), v.numpy(), _lut(mask), 64, 64)
    want = oa.dense_masked_attention(q, k, v, mask).numpy()
    assert np.abs(got - want).max() < 2e-5


def test_block_all_full_equals_sdpa_and_causal():
    s = 128
    q, k, v = _qkv(1, 2, s, 64, seed=5)
    got = oa.block_attn_mask(q.numpy(), k.numpy(), v.numpy(), _lut(torch.ones(s, s)), 64, 64)
    assert np.abs(got - F.scaled_dot_product_attention(q, k, v).numpy()).max() < 2e-5
    got = oa.block_attn_mask(q.numpy(), k.numpy(), v.numpy(), _lut(torch.tril(torch.ones(s, s)), 32, 32), 32, 32)
    assert np.abs(got - F.scaled_dot_product_attention(q, k, v, is_causal=True).numpy()).max() < 2e-5


def test_block_key_block_order_invariance_and_unit_v():
    s = 256
    mask = configs.mask_c5(s)
    q, k, v = _qkv(1, 1, s, 64, seed=6)
    lut = list(_lut(mask))
    base = oa.block_attn_mask(q.numpy(), k.numpy(), v.numpy(), tuple(lut), 64, 64)
    # reverse each row's LOAD order (FULL / PART lists reversed consistently)
    def rev(rp, ci, extra=None):
        ci = ci.copy(); ex = None if extra is None else extra.copy()
        for r in range(len(rp) - 1):
            ci[rp[r]:rp[r + 1]] = ci[rp[r]:rp[r + 1]][::-1]
            if ex is not None:
                ex[rp[r]:rp[r + 1]] = ex[rp[r]:rp[r + 1]][::-1]
        return ci, ex
    lut[2], _ = rev(lut[1], lut[2])
    lut[4], lut[5] = rev(lut[3], lut[4], lut[5])
    lut[7], _ = rev(lut[6], lut[7])
    # the merge walk needs FULL and PART each in LOAD order: reversed lists satisfy that
    perm = oa.block_attn_mask(q.numpy(), k.numpy(), v.numpy(), tuple(lut), 64, 64)
    assert np.abs(perm - base).max() < 2e-5
    ones = oa.block_attn_mask(q.numpy(), k.numpy(), np.ones_like(v.numpy()), _lut(mask), 64, 64)
    assert np.abs(ones - 1).max() < 1e-5        # probabilities sum to one


def test_block_dead_rows_and_empty_query_block_are_zero():
    s = 128
    mask = torch.ones(s, s)
    mask[64:, :] = 0            # second query block has no LUT entry at all
    mask[3, :] = 0              # a dead row inside a live block
    q, k, v = _qkv(1, 1, s, 64, seed=7)
    got = oa.block_attn_mask(q.numpy(), k.numpy(), v.numpy(), _lut(mask), 64, 64)
    assert np.all(got[0, 0, 64:] == 0) and np.all(got[0, 0, 3] == 0)
    assert np.abs(got - oa.dense_masked_attention(q, k, v, mask).numpy()).max() < 2e-5


def test_rowwise_oracles():
    s = 96
    q, k, v = _qkv(2, 3, s, 64, seed=8)
    merge = lambda o: o.permute(0, 2, 1, 3).reshape(2, s, 3 * 64)
    assert torch.allclose(oa.rowwise_attn_full(q, k, v, False), merge(F.scaled_dot_product_attention(q, k, v)), atol=2e-6)
    assert torch.allclose(oa.rowwise_attn_full(q, k, v, True),
                          merge(F.scaled_dot_product_attention(q, k, v, is_causal=True)), atol=2e-6)
    i = torch.arange(s)[:, None]; j = torch.arange(s)[None, :]
    band = 7
    allowed = (j > i - band) & (j <= i)
    assert torch.allclose(oa.rowwise_attn_sliding(q, k, v, True, band),
                          merge(F.scaled_dot_product_attention(q, k, v, attn_mask=allowed)), atol=2e-6)
    rm = (torch.rand(s, s, generator=torch.Generator().manual_seed(1)) < 0.5).half()
    rm[:, 0] = 1
    assert torch.allclose(oa.rowwise_attn_mask(q, k, v, False, rm),
                          merge(F.scaled_dot_product_attention(q, k, v, attn_mask=rm > 0)), atol=2e-6)
