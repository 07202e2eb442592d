"""GPU parity of the fused encoder operators on bfloat16 tensors (the reference computes in fp16
only; this format is an addition behind the same operators) against the CPU oracle in fp32 on the
same bf16-rounded inputs.

Tolerance: bfloat16 keeps 8 significant bits, so a stored result carries a relative rounding
error of 2^-9 where fp16 carries 2^-12:
    |got - want| <= 8e-3 + 1.6e-2 * |want|
(the bound of the bfloat16 attention tests).  A stack of layers is checked against the same
stack in plain PyTorch ops on bfloat16 tensors instead, with the bound stated there.
"""
import pytest
import torch

from oracle import encoder as oe
from stof import configs, fused, masks as pm
from stof.fused import StofError
from stof.layer import EncoderLayer, eager_layer

pytestmark = pytest.mark.gpu
ATOL, RTOL = 8e-3, 1.6e-2
BF = torch.bfloat16


def _close(got, want, what=""):
    assert got.dtype == BF
    got = got.float().cpu(); want = want.float().cpu()
    assert got.shape == want.shape
    err = (got - want).abs()
    bad = err > ATOL + RTOL * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements out of tolerance, max abs err {float(err.max()):.3e}"
    print(f"{what}: max abs err {float(err.max()):.3e}", flush=True)


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(BF)


# (8192, 3072, 768) / (8155, 3080, 1024): the 128 x 128 form, full and ragged; (300, 768, 3072): the
# 64-token form with K split (the library's rule); (64, 2304, 768), (129, 136, 128): the 64-token form
@pytest.mark.parametrize("M,N,K", [(8192, 3072, 768), (8155, 3080, 1024), (300, 768, 3072), (64, 2304, 768), (129, 136, 128)])
@pytest.mark.parametrize("act", ["none", "gelu", "gelu_tanh", "relu"])
def test_gemm_bias_act_bf16(M, N, K, act):
    print(f"bf16 gemm M{M} N{N} K{K} {act}", flush=True)
    x = _rand(M, K, seed=1); W = _rand(K, N, seed=2, scale=0.05); b = _rand(N, seed=3, scale=0.5)
    got = fused.gemm_bias_act(x.cuda(), fused.pack_weight(W.cuda()), b.cuda(), act)
    _close(got, oe.gemm_bias_act(x, W, b, act), f"gemm {act}")


@pytest.mark.parametrize("splits", [2, 3])
def test_gemm_split_k_bf16(splits):
    for (M, N, K) in [(512, 768, 3072), (3072, 768, 3072)]:       # the 64-token form and the 128 x 128 form
        x = _rand(M, K, seed=4); W = _rand(K, N, seed=5, scale=0.05); b = _rand(N, seed=6, scale=0.5)
        xg, Wt, bg = x.cuda(), fused.pack_weight(W.cuda()), b.cuda()
        got = fused.gemm_bias_act(xg, Wt, bg, "gelu", splits=splits)
        _close(got, oe.gemm_bias_act(x, W, b, "gelu"), f"split-K {splits} M{M}")
        assert torch.equal(fused.gemm_bias_act(xg, Wt, bg, "gelu", splits=splits), got)


@pytest.mark.parametrize("M,N", [(8192, 768), (1000, 1024), (7, 256), (300, 4096)])
def test_bias_residual_layernorm_bf16(M, N):
    x = _rand(M, N, seed=7); b = _rand(N, seed=8, scale=0.5); r = _rand(M, N, seed=9)
    gm = (1 + 0.1 * _rand(N, seed=10).float()).to(BF); bt = _rand(N, seed=11, scale=0.1)
    got = fused.bias_residual_layernorm(x.cuda(), b.cuda(), r.cuda(), gm.cuda(), bt.cuda(), 1e-5)
    want = oe.layer_norm(x.float() + b.float() + r.float(), gm.float(), bt.float(), 1e-5)
    _close(got, want, "bias + residual + LN")
    got = fused.bias_residual_layernorm(x.cuda(), None, None, None, None, 1e-5)
    _close(got, oe.layer_norm(x.float(), eps=1e-5), "LN alone")


# cluster form (8192 rows; 3000 x 384: three workgroups per row block), two launches (300 rows)
@pytest.mark.parametrize("M,N,K", [(8192, 768, 768), (8192, 1024, 4096), (3000, 384, 192), (300, 768, 3072)])
@pytest.mark.parametrize("form", ["auto", "cluster", "split"])
def test_gemm_bias_residual_layernorm_bf16(M, N, K, form):
    print(f"bf16 gemm_ln M{M} N{N} K{K} {form}", flush=True)
    x = _rand(M, K, seed=12); W = _rand(K, N, seed=13, scale=0.05); b = _rand(N, seed=14, scale=0.5)
    r = _rand(M, N, seed=15); gm = (1 + 0.1 * _rand(N, seed=16).float()).to(BF); bt = _rand(N, seed=17, scale=0.1)
    got = fused.gemm_bias_residual_layernorm(x.cuda(), fused.pack_weight(W.cuda()), b.cuda(), r.cuda(), gm.cuda(), bt.cuda(), 1e-5, form=form)
    assert not fused.cluster_exchange_failed()
    _close(got, oe.gemm_bias_residual_layernorm(x, W, b, r, gm, bt, 1e-5), f"gemm_ln {form}")


def test_bf16_argument_checks():
    x = _rand(64, 128).cuda(); W = _rand(256, 128).cuda()
    with pytest.raises(StofError):
        fused.gemm_bias_act(x, W.half(), None, "none")                      # mixed formats
    with pytest.raises(StofError):
        fused.gemm_bias_act(x, W, _rand(256).cuda().half(), "none")
    with pytest.raises(StofError):
        fused.gemm_bias_residual_layernorm(x, W, None, None, None, None, form="row")     # the row form is fp16 only
    with pytest.raises(StofError):
        fused.gemm_act_gemm(x, W, None, _rand(128, 256).cuda())               # the chained kernel is fp16 only
    with pytest.raises(StofError):
        fused.bias_residual_layernorm(x.float(), None, None, None, None)


@pytest.mark.parametrize("gelu", ["erf", "tanh", "relu"])
def test_encoder_layer_bf16(gelu):
    """One BERT-base layer at B4 S512 (hidden 768: both LayerNorm GEMMs in their cluster form) on
    bfloat16 tensors against the fp32 oracle: five kernels, each storing 8 significant bits, on
    normalised outputs of magnitude up to 4 - bound 3e-2 + 3e-2 |want| (observed max abs error 2.6e-2 .. 2.9e-2;
    the same layer in plain PyTorch ops on the same bfloat16 tensors: 4.2e-2 .. 4.6e-2)."""
    B, S, D, H, F = 4, 512, 768, 12, 3072
    w = configs.layer_weights(D, F, seed=0)
    wb = {k: v.to(BF) for k, v in w.items()}
    x = configs.layer_input(configs.LayerConfig("t", B, S, D, H, F, 1), seed=1).to(BF)
    mask = configs.mask_c1(S)[None]
    lut = pm.get_sparse_storage(mask.float().cuda(), 64, 64)[1:]
    layer = EncoderLayer({k: v.cuda() for k, v in wb.items()}, H, eps=1e-12, gelu=gelu)
    got = layer(x.cuda(), lut)
    assert got.dtype == BF and got.shape == x.shape
    want = oe.bert_layer(x.float(), {k: v.float() for k, v in wb.items()}, mask.float(), H, eps=1e-12, gelu=gelu)
    err = (got.float().cpu() - want).abs()
    bad = err > 3e-2 + 3e-2 * want.abs()
    assert not bool(bad.any()), f"{int(bad.sum())} elements out of tolerance, max abs err {float(err.max()):.3e}"
    print(f"bf16 layer {gelu}: max abs err {float(err.max()):.3e}", flush=True)
    # and the same layer in plain PyTorch ops on the same bfloat16 tensors is no closer to the oracle
    eager = eager_layer(x.cuda(), {k: v.cuda() for k, v in wb.items()}, mask.cuda().to(BF), H, 1e-12, gelu=gelu)
    err_eager = (eager.float().cpu() - want).abs().max().item()
    print(f"   plain PyTorch ops on bf16: max abs err {err_eager:.3e}", flush=True)
    assert float(err.max()) <= max(2.0 * err_eager, 3e-2)
