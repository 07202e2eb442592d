"""Pins the CPU oracle of the mask generators and the LUT compiler (oracle/masks.py)
without the reference: closed-form predicates, exhaustive brute force, round trip,
hand-derived block counts - and checks the product's vectorised torch implementation
(stof.masks) bit for bit against the oracle."""
import itertools
import random

import numpy as np
import pytest
import torch

from oracle import masks as om
from stof import masks as pm
from stof import configs


def _attr(b, s):
    return np.ones((b, s, s), dtype=np.float32)


# ---- generators: independent closed forms, element by element -----------------------------

def _pred_mask(b, s, pred, causal):
    m = np.zeros((b, s, s), dtype=np.float32)
    for bb in range(b):
        for i in range(s):
            for j in range(s):
                ok = pred(i, j)
                if causal and bb == b - 1 and j > i:   # the trim reaches the last batch only
                    ok = False
                m[bb, i, j] = 1.0 if ok else 0.0
    return m


@pytest.mark.parametrize("b,s,bw,causal", [(1, 16, 1, False), (2, 24, 3, True), (1, 33, 5, True), (3, 8, 0, True)])
def test_sliding_closed_form(b, s, bw, causal):
    want = _pred_mask(b, s, lambda i, j: abs(i - j) <= bw, causal)
    assert np.array_equal(om.generate_sliding_mask(_attr(b, s), bw, causal), want)


@pytest.mark.parametrize("b,s,bw,d,causal", [(1, 16, 1, 1, False), (2, 24, 4, 1, True), (1, 32, 3, 2, True), (1, 20, 2, 3, False)])
def test_dilated_closed_form(b, s, bw, d, causal):
    def pred(i, j):
        w = bw + d
        return i - w <= j < min(s, i + w + 1) and (j - (i - w)) % (d + 1) == 0
    want = _pred_mask(b, s, pred, causal)
    assert np.array_equal(om.generate_dilated_mask(_attr(b, s), bw, d, causal), want)


@pytest.mark.parametrize("b,s,g,bw,causal", [(1, 16, 2, 1, False), (2, 32, 3, 2, True), (1, 30, 4, 0, False)])
def test_longformer_closed_form(b, s, g, bw, causal):
    lo, hi = int(s / 2), int(s / 2 + g)
    pred = lambda i, j: i < g or j < g or lo <= i < hi or lo <= j < hi or abs(i - j) <= bw
    want = _pred_mask(b, s, pred, causal)
    assert np.array_equal(om.generate_longformer_mask(_attr(b, s), g, bw, causal), want)


def test_causal_is_tril():
    m = om.generate_causal_mask(_attr(2, 9))
    assert m.shape == (2, 9, 9) and np.array_equal(m[1], np.tril(np.ones((9, 9))))


def test_bigbird_structure_and_rng_order():
    """global + band part is a closed form; the random part must be exactly the points an
    independently written replay of the documented draw order produces."""
    b, s, g, bw, fill = 2, 128, 4, 2, 0.1
    m = om.generate_bigbird_mask(_attr(b, s), g, bw, fill, False)
    base = _pred_mask(b, s, lambda i, j: i < g or j < g or abs(i - j) <= bw, False)
    assert np.all(m >= base)
    rng = random.Random(0)      # same Mersenne Twister stream as random.seed(0)
    pts = np.zeros_like(base)
    nblk = s // 32
    for bb in range(b):
        for blk in range(nblk - 1):
            if blk == 0:
                off = rng.choice([1, 0])
            elif blk == nblk - 2:
                off = rng.choice([-1, 0])
            else:
                off = rng.choice([-1, 0, 1])
            for _ in range(int(1024 * fill)):
                x = rng.randint(0, 32); y = rng.randint(0, 32)
                pts[bb, blk * 32 + x, (blk + off) * 32 + y] = 1
    assert np.array_equal(m, np.maximum(base, pts))


# ---- LUT compiler --------------------------------------------------------------------------

def _classify_independent(mask2d, bm, bn):
    """Independent classifier: counts ones per block."""
    n = mask2d.shape[0]
    out = {}
    for r in range(n // bm):
        for c in range(n // bn):
            ones = int(mask2d[r * bm:(r + 1) * bm, c * bn:(c + 1) * bn].sum())
            out[(r, c)] = "full" if ones == bm * bn else ("empty" if ones == 0 else "part")
    return out


def _check_lut_against_classes(lut, mask2d, bm, bn):
    _, frp, fci, prp, pci, pbm, lrp, lci = lut
    cls = _classify_independent(mask2d, bm, bn)
    nq, nk = mask2d.shape[0] // bm, mask2d.shape[0] // bn
    pslot = 0
    for r in range(nq):
        full = [c for c in range(nk) if cls[(r, c)] == "full"]
        part = [c for c in range(nk) if cls[(r, c)] == "part"]
        assert list(fci[frp[r]:frp[r + 1]]) == full
        assert list(pci[prp[r]:prp[r + 1]]) == part
        assert list(lci[lrp[r]:lrp[r + 1]]) == sorted(full + part)
        for c in part:
            blk = mask2d[r * bm:(r + 1) * bm, c * bn:(c + 1) * bn]
            want = np.where(blk == 1, np.float16(0), np.float16(-10000))
            assert pbm[pslot].dtype == np.float16 and np.array_equal(pbm[pslot], want)
            pslot += 1
    assert frp[0] == prp[0] == lrp[0] == 0
    assert frp[-1] == len(fci) and prp[-1] == len(pci) and lrp[-1] == len(lci)
    assert all(a.dtype == np.int32 for a in (frp, fci, prp, pci, lrp, lci))
    if pslot == 0:
        assert pbm.shape == (1, bm, bn) and np.all(pbm == 1)
    else:
        assert pbm.shape == (pslot, bm, bn)


def test_lut_bruteforce_all_masks_2x2_blocks():
    """Every one of the 2^16 0/1 masks on a 4x4 grid with 2x2 blocks."""
    for bits in range(1 << 16):
        m = np.array([(bits >> t) & 1 for t in range(16)], dtype=np.float32).reshape(1, 4, 4)
        lut = om.get_sparse_storage(m, 2, 2)
        if bits % 257 == 0 or bits < 64:          # full structural check on a subset (speed)
            _check_lut_against_classes(lut, m[0], 2, 2)
        assert np.array_equal(om.expand_sparse_storage(lut, 4, 2, 2), m[0])
        assert abs(float(lut[0]) - 100.0 * bin(bits).count("1") / 16) < 1e-4


@pytest.mark.parametrize("bm,bn", [(16, 16), (32, 16), (16, 64), (64, 64)])
def test_lut_random_masks_roundtrip_and_classes(bm, bn):
    rng = np.random.default_rng(bm * 131 + bn)
    n = 128
    blk = rng.integers(0, 3, size=(n // bm, n // bn))
    m = np.zeros((2, n, n), dtype=np.float32)
    for r in range(n // bm):
        for c in range(n // bn):
            if blk[r, c] == 1:
                m[0, r * bm:(r + 1) * bm, c * bn:(c + 1) * bn] = 1
            elif blk[r, c] == 2:
                m[0, r * bm:(r + 1) * bm, c * bn:(c + 1) * bn] = rng.integers(0, 2, size=(bm, bn))
    m[1] = 1 - m[0]    # batch 1 must be ignored by the LUT (batch 0 only) but counted in nnz
    lut = om.get_sparse_storage(m, bm, bn)
    _check_lut_against_classes(lut, m[0], bm, bn)
    assert np.array_equal(om.expand_sparse_storage(lut, n, bm, bn), m[0])
    assert abs(float(lut[0]) - 100.0 * m.sum() / (n * n)) < 1e-3


@pytest.mark.parametrize("name", ["C1", "C2", "C4", "C5"])
def test_config_block_counts_known_answers(name):
    """Hand-derived counts of full / partial 64x64 blocks for the benchmark masks."""
    mask = configs.ATTN_MASKS[name]().numpy().astype(np.float32)[None]
    lut = om.get_sparse_storage(mask, 64, 64)
    nfull, npart = configs.BLOCK_COUNTS[name]
    assert (len(lut[2]), len(lut[4])) == (nfull, npart)
    assert len(lut[7]) == nfull + npart


def test_minus_10000_is_exact_in_fp16():
    assert float(np.float16(-10000.0)) == -10000.0


# ---- product implementation (torch, vectorised) == oracle, bit for bit --------------------

def _same_lut(p, o):
    assert abs(float(p[0]) - float(o[0])) < 1e-3
    for a, b in zip(p[1:], o[1:]):
        a = a.cpu().numpy()
        assert a.dtype == b.dtype and a.shape == b.shape and np.array_equal(a, b)


@pytest.mark.parametrize("gen,kwargs", [
    ("generate_sliding_mask", dict(bandwidth=32, is_cauasl=True)),
    ("generate_sliding_mask", dict(bandwidth=5, is_cauasl=False)),
    ("generate_dilated_mask", dict(bandwidth=32, dilation_rate=1, is_cauasl=True)),
    ("generate_dilated_mask", dict(bandwidth=7, dilation_rate=3, is_cauasl=False)),
    ("generate_longformer_mask", dict(globalwidth=32, bandwidth=32, is_cauasl=False)),
    ("generate_longformer_mask", dict(globalwidth=3, bandwidth=9, is_cauasl=True)),
    ("generate_bigbird_mask", dict(globalwidth=32, bandwidth=32, fill_rate=0.1, is_cauasl=False)),
    ("generate_bigbird_mask", dict(globalwidth=8, bandwidth=4, fill_rate=0.05, is_cauasl=True)),
])
@pytest.mark.parametrize("b,s", [(1, 128), (2, 256)])
def test_product_generators_equal_oracle(gen, kwargs, b, s):
    attr = torch.ones(b, s, s, dtype=torch.float16)
    got = getattr(pm, gen)(attr, **kwargs)
    want = getattr(om, gen)(np.ones((b, s, s), dtype=np.float16), **kwargs)
    assert got.dtype == attr.dtype and got.shape == attr.shape
    assert np.array_equal(got.numpy(), want)
    for blk in (16, 32, 64):
        _same_lut(pm.get_sparse_storage(got, blk, blk), om.get_sparse_storage(want, blk, blk))


def test_product_causal_mask():
    attr = torch.ones(3, 40, 40, dtype=torch.float16)
    got = pm.generate_causal_mask(attr)
    assert got.dtype == torch.float32 and got.device.type == "cpu"
    assert np.array_equal(got.numpy(), om.generate_causal_mask(attr.numpy()))


@pytest.mark.parametrize("bm,bn", [(16, 16), (32, 64), (64, 32), (64, 64)])
def test_product_lut_random_equal_oracle(bm, bn):
    rng = np.random.default_rng(7 + bm + bn)
    n = 256
    dense = (rng.random((2, n, n)) < 0.5).astype(np.float32)
    # carve empty and full blocks so that all three classes appear
    dense[0, :64, :128] = 0
    dense[0, 64:192, 64:192] = 1
    _same_lut(pm.get_sparse_storage(torch.from_numpy(dense), bm, bn), om.get_sparse_storage(dense, bm, bn))
    # fp16 input, as the reference's callers pass it
    _same_lut(pm.get_sparse_storage(torch.from_numpy(dense).half(), bm, bn),
              om.get_sparse_storage(dense.astype(np.float16), bm, bn))


def test_product_lut_edge_cases():
    n = 128
    ones = torch.ones(1, n, n)
    lut = pm.get_sparse_storage(ones, 64, 64)          # no partial block: dummy ones block
    assert lut[5].shape == (1, 64, 64) and bool((lut[5] == 1).all()) and lut[4].numel() == 0
    _same_lut(lut, om.get_sparse_storage(ones.numpy(), 64, 64))
    zeros = torch.zeros(1, n, n)                        # nothing active: empty column lists
    lut = pm.get_sparse_storage(zeros, 64, 64)
    assert lut[7].numel() == 0 and lut[6].tolist() == [0, 0, 0]
    _same_lut(lut, om.get_sparse_storage(zeros.numpy(), 64, 64))
    with pytest.raises(ValueError):
        pm.get_sparse_storage(torch.ones(1, 100, 100), 64, 64)   # ragged: rejected loudly


def test_product_expand_roundtrip_and_batched():
    m3, L = configs.mask_c3(batch=4, s=256, window=64, seed=3)
    m3 = m3.float()
    lutb = pm.get_sparse_storage_batched(m3, 64, 64)
    nq = 4
    for b in range(4):
        single = pm.get_sparse_storage(m3[b:b + 1], 64, 64)
        frp, fci, prp, pci, pbm, lrp, lci = lutb[1:]
        for (rp, ci, srp, sci) in ((frp, fci, single[1], single[2]), (prp, pci, single[3], single[4]),
                                   (lrp, lci, single[6], single[7])):
            base = int(rp[b, 0])
            assert torch.equal(rp[b] - base, srp)
            assert torch.equal(ci[base:int(rp[b, -1])], sci)
        if single[4].numel():
            assert torch.equal(pbm[int(prp[b, 0]):int(prp[b, -1])], single[5])
        assert torch.equal(pm.expand_sparse_storage(single, 256, 64, 64), m3[b])
    one = pm.get_sparse_storage_batched(m3[:1], 64, 64)
    ref = pm.get_sparse_storage(m3[:1], 64, 64)
    for a, b_ in zip(one[1:], ref[1:]):
        assert torch.equal(a.reshape(b_.shape), b_)


# ---- golden vectors produced by the reference's own bigbird generator ----------------------

def test_bigbird_golden_from_reference():
    """tests/golden/bigbird_ref.npz was written by tests/golden/make_bigbird_fixture.py, which
    ran the reference's generate_bigbird_mask; the oracle and the product must reproduce it."""
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "bigbird_ref.npz")
    z = np.load(path)
    cases = json.loads(bytes(z["cases"]).decode())
    for n, c in enumerate(cases):
        b, s = c["batch"], c["seq"]
        want = np.unpackbits(z[f"mask{n}"])[: b * s * s].reshape(b, s, s).astype(np.float32)
        kw = dict(globalwidth=c["globalwidth"], bandwidth=c["bandwidth"], fill_rate=c["fill_rate"],
                  is_cauasl=c["is_cauasl"])
        assert np.array_equal(om.generate_bigbird_mask(np.ones((b, s, s), dtype=np.float32), **kw), want)
        got = pm.generate_bigbird_mask(torch.ones(b, s, s, dtype=torch.float16), **kw)
        assert np.array_equal(got.float().numpy(), want)
