"""Pins the encoder oracle (oracle/encoder.py) with library routines and closed forms."""
import math

import torch
import torch.nn.functional as F

from oracle import encoder as oe
from stof import configs


def _r(*s, seed=0, scale=1.0):
    return torch.randn(*s, generator=torch.Generator().manual_seed(seed)) * scale


def test_layer_norm_matches_library_and_closed_form():
    x = _r(5, 7, 96, seed=1) * 3 + 2
    g, b = 1 + 0.1 * _r(96, seed=2), _r(96, seed=3)
    for eps in (1e-5, 1e-12):
        assert torch.allclose(oe.layer_norm(x, g, b, eps), F.layer_norm(x, (96,), g, b, eps), atol=1e-5)
    y = oe.layer_norm(x, eps=0.0)
    assert float(y.mean(-1).abs().max()) < 1e-6 and float((y.var(-1, unbiased=False) - 1).abs().max()) < 1e-5
    x64 = x.double()
    m = x64.mean(-1, keepdim=True)
    ref = (x64 - m) / torch.sqrt(((x64 - m) ** 2).mean(-1, keepdim=True) + 1e-5)
    assert torch.allclose(oe.layer_norm(x, eps=1e-5).double(), ref, atol=1e-5)


def test_gelus():
    x = _r(1000, seed=4) * 3
    assert torch.allclose(oe.new_gelu(x), F.gelu(x, approximate="tanh"), atol=1e-6)
    assert torch.allclose(oe.gemm_bias_act(torch.eye(8), torch.eye(8), torch.zeros(8), "gelu"),
                          F.gelu(torch.eye(8)), atol=1e-7)
    erf = 0.5 * x * (1 + torch.erf(x / math.sqrt(2)))
    assert torch.allclose(F.gelu(x), erf, atol=1e-6)


def test_fused_op_oracles():
    A = _r(2, 9, 32, seed=5); W = _r(32, 48, seed=6, scale=0.2); bias = _r(48, seed=7)
    got = oe.matmul_bias_layernorm(A, W.expand(2, -1, -1), bias)
    assert torch.allclose(got, F.layer_norm(A @ W + bias, (48,)), atol=1e-5)
    res = _r(2, 9, 48, seed=8)
    got = oe.matmul_bias_layernorm(A, W.expand(2, -1, -1), bias + res)
    assert torch.allclose(got, F.layer_norm(A @ W + bias + res, (48,)), atol=1e-5)
    x = _r(3, 5, 48, seed=9); w = _r(48, seed=10); b = _r(48, seed=11)
    assert torch.allclose(oe.batched_bias_layernorm(x, bias, w, b), F.layer_norm(x + bias, (48,), w, b), atol=1e-5)
    # W = I, zero bias/residual: plain LayerNorm of the input
    eye = torch.eye(48)
    got = oe.gemm_bias_residual_layernorm(x, eye, torch.zeros(48), torch.zeros_like(x), w, b)
    assert torch.allclose(got, F.layer_norm(x, (48,), w, b), atol=1e-5)
    a = _r(2, 6, 16, seed=12); b1 = _r(16, 64, seed=13, scale=0.3); d = _r(64, 16, seed=14, scale=0.3); bb = _r(64, seed=15)
    t = F.gelu(a @ b1 + bb, approximate="tanh").half().float()
    assert torch.allclose(oe.matmul_gelu_matmul(a, b1, d, bb), t @ d, atol=1e-5)


def test_bert_layer_against_module_style_evaluation():
    """The layer oracle against an independent evaluation with torch modules' functional forms
    (F.scaled_dot_product_attention, F.linear, F.layer_norm, F.gelu)."""
    B, S, D, H, Fd = 2, 64, 64, 4, 128
    w = configs.layer_weights(D, Fd, seed=3, dtype=torch.float32)
    x = _r(B, S, D, seed=16)
    mask = torch.tril(torch.ones(S, S))[None].expand(B, -1, -1)
    got = oe.bert_layer(x, w, mask, H, eps=1e-12)
    qkv = F.linear(x, w["W_qkv"].t(), w["b_qkv"])
    q, k, v = (t.view(B, S, H, D // H).transpose(1, 2) for t in qkv.chunk(3, -1))
    a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, S, D)
    h = F.layer_norm(F.linear(a, w["W_o"].t(), w["b_o"]) + x, (D,), w["g1"], w["be1"], 1e-12)
    f = F.gelu(F.linear(h, w["W_1"].t(), w["b_1"]))
    want = F.layer_norm(F.linear(f, w["W_2"].t(), w["b_2"]) + h, (D,), w["g2"], w["be2"], 1e-12)
    assert torch.allclose(got, want, atol=2e-5)
    # pre-made QKV activation variant (the reference's layer has no QKV GEMM)
    w2 = dict(w); w2["W_qkv"] = None; w2["qkv_act"] = x @ w["W_qkv"]
    assert torch.allclose(oe.bert_layer(x, w2, mask, H, eps=1e-12), want, atol=2e-5)


def test_bert_layer_fp16_rounding_points_and_activations():
    """round_fp16 is pinned by an independent evaluation with explicit .half() stores at the
    five operator boundaries (and, for "split", after the two products that feed a
    LayerNorm); relu / tanh against F.relu / F.gelu(approximate="tanh")."""
    B, S, D, H, Fd = 2, 64, 64, 4, 128
    w = configs.layer_weights(D, Fd, seed=5, dtype=torch.float16)
    wf = {k: v.float() for k, v in w.items()}
    x = _r(B, S, D, seed=17).half()
    mask = torch.tril(torch.ones(S, S))[None].expand(B, -1, -1)
    h16 = lambda t: t.half().float()
    for mode in (True, "split"):
        for act, fn in (("erf", F.gelu), ("tanh", lambda t: F.gelu(t, approximate="tanh")), ("relu", F.relu)):
            got = oe.bert_layer(x, w, mask, H, eps=1e-12, gelu=act, round_fp16=mode)
            qkv = h16(F.linear(x.float(), wf["W_qkv"].t(), wf["b_qkv"]))
            q, k, v = (t.view(B, S, H, D // H).transpose(1, 2) for t in qkv.chunk(3, -1))
            a = h16(F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, S, D))
            p1 = F.linear(a, wf["W_o"].t())
            p1 = h16(p1) if mode == "split" else p1
            h = h16(F.layer_norm(p1 + wf["b_o"] + x.float(), (D,), wf["g1"], wf["be1"], 1e-12))
            f = h16(fn(F.linear(h, wf["W_1"].t(), wf["b_1"])))
            p2 = F.linear(f, wf["W_2"].t())
            p2 = h16(p2) if mode == "split" else p2
            want = h16(F.layer_norm(p2 + wf["b_2"] + h, (D,), wf["g2"], wf["be2"], 1e-12))
            # equal up to the last place of fp16 where the two evaluations' fp32 sums differ in order
            assert float((got - want).abs().max()) <= 2e-3, (mode, act)
            assert torch.equal(got, h16(got))                    # the result is an fp16 value
    # and the rounding moves the layer's result by less than the comparison tolerance
    ref = oe.bert_layer(x, w, mask, H, eps=1e-12)
    assert 0 < float((oe.bert_layer(x, w, mask, H, eps=1e-12, round_fp16=True) - ref).abs().max()) < 4e-3
