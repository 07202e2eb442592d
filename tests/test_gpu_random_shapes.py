"""Seeded sweeps over shapes that no hand-picked case names: the GEMM entry points pick among four
launch forms (64-token ring, 128 x 128, each with or without K split over workgroups) and the
LayerNorm GEMM among three, by rules on the shape; every draw is checked against the CPU oracle.
Tolerance as in the other operator tests: 2e-3 + 1e-2 |want| for fp16, 8e-3 + 1.6e-2 |want| for
bfloat16 (8 significant bits in the stored result)."""
import random

import pytest
import torch

from oracle import attention as oa
from oracle import encoder as oe
from stof import fused, masks as pm
from stof.ops import block_attn

pytestmark = pytest.mark.gpu
TOL = {torch.float16: (2e-3, 1e-2), torch.bfloat16: (8e-3, 1.6e-2)}


def _close(got, want, what):
    atol, rtol = TOL[got.dtype]
    got = got.float().cpu(); want = want.float().cpu()
    assert got.shape == want.shape
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} out of tolerance, max abs err {float(err.max()):.3e}"


def _rand(shape, gen, dtype, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


@pytest.mark.parametrize("seed", range(24))
def test_gemm_bias_act_random_shapes(seed):
    rnd = random.Random(1000 + seed)
    M = rnd.choice([1, 3, 64, 65, 127, 200, 511, 777, 1030, 2049, 3000, 4097])
    N = 8 * rnd.randint(1, 260)
    K = 64 * rnd.randint(1, 50)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    act = rnd.choice(["none", "gelu", "gelu_tanh", "relu"])
    splits = rnd.choice([None, None, 1, 2, 5])
    print(f"gemm M{M} N{N} K{K} {dtype} {act} splits {splits}", flush=True)
    g = torch.Generator().manual_seed(seed)
    x = _rand((M, K), g, dtype, 0.5); W = _rand((K, N), g, dtype, 0.05); b = _rand((N,), g, dtype, 0.5)
    got = fused.gemm_bias_act(x.cuda(), fused.pack_weight(W.cuda()), b.cuda() if seed % 5 else None, act, splits=splits)
    _close(got, oe.gemm_bias_act(x, W, b if seed % 5 else torch.zeros(N), act), f"gemm seed {seed}")


@pytest.mark.parametrize("seed", range(16))
def test_gemm_layernorm_random_shapes(seed):
    rnd = random.Random(2000 + seed)
    M = rnd.choice([5, 128, 300, 1000, 2048, 3333, 6000, 9000])
    N = 128 * rnd.randint(2, 8)
    K = 64 * rnd.randint(1, 40)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    form = rnd.choice(["auto", "auto", "cluster", "split"])
    eps = rnd.choice([1e-5, 1e-12])
    print(f"gemm_ln M{M} N{N} K{K} {dtype} {form} eps {eps}", flush=True)
    g = torch.Generator().manual_seed(seed)
    x = _rand((M, K), g, dtype, 0.5); W = _rand((K, N), g, dtype, 0.05); b = _rand((N,), g, dtype, 0.5)
    r = _rand((M, N), g, dtype); gm = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype); bt = _rand((N,), g, dtype, 0.1)
    got = fused.gemm_bias_residual_layernorm(x.cuda(), fused.pack_weight(W.cuda()), b.cuda(), r.cuda(), gm.cuda(), bt.cuda(), eps, form=form)
    assert not fused.cluster_exchange_failed()
    _close(got, oe.gemm_bias_residual_layernorm(x, W, b, r, gm, bt, eps), f"gemm_ln seed {seed}")


@pytest.mark.parametrize("seed", range(12))
def test_block_attention_random_masks(seed):
    """Random block structure (empty, full and partial tiles at random, some rows without any key)
    on random batch / head counts, both element formats, every launch form."""
    rnd = random.Random(3000 + seed)
    S = 64 * rnd.randint(1, 12)
    B, H = rnd.randint(1, 3), rnd.randint(1, 5)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    form = rnd.choice([None, "two_rows", "key_split", "pipelined"])
    g = torch.Generator().manual_seed(seed)
    nb = S // 64
    kind = torch.randint(0, 3, (nb, nb), generator=g)          # 0 empty, 1 full, 2 partial
    mask = torch.zeros(S, S, dtype=torch.bool)
    for r in range(nb):
        for c in range(nb):
            blk = mask[64 * r:64 * r + 64, 64 * c:64 * c + 64]
            if kind[r, c] == 1:
                blk[:] = True
            elif kind[r, c] == 2:
                blk[:] = torch.rand(64, 64, generator=g) < rnd.choice([0.02, 0.5, 0.98])
    if S > 64:
        mask[rnd.randrange(S)] = False                          # a query without keys
    print(f"attention B{B} H{H} S{S} {dtype} {form}", flush=True)
    q, k, v = (_rand((B, H, S, 64), g, dtype).cuda() for _ in range(3))
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    got = block_attn(q, k, v, lut, 64, 64, launch_form=form)
    want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask)
    _close(got, want, f"attention seed {seed}")
