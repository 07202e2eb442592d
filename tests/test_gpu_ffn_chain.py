"""GPU parity of the single-launch chained GEMM + bias + activation + GEMM (stof_gemm_act_gemm,
the replacement of triton_matmul_batch, src/triton_template/gemm_gemm.py:99-174) against the CPU
oracle, which rounds the intermediate to fp16 as the reference kernel does (gemm_gemm.py:152).

Tolerance: |got - want| <= 2e-3 + 1e-2 |want| (fp16 output of fp32 sums over F = 3072 terms;
observed max abs error 3.9e-3 at (1, 512, 768, 3072) = one fp16 ulp of results of magnitude 4 to
8).  The contributions of the F / 128 chunks are added with fp32 atomics, so two runs may differ
in the last bit of an fp16 result; comparisons between runs allow one fp16 ulp.

The single-launch form is NOT the faster one on MI355X (67 us against 31 us for two launches at
this size); it is opt-in, and the first test prints both times.
"""
import pytest
import torch

from oracle import encoder as oe
from stof import configs, fused, masks as pm
from stof.layer import EncoderLayer
from stof.ops import StofError

pytestmark = pytest.mark.gpu


def _close(got, want, what="", atol=2e-3, rtol=1e-2):
    got = got.float().cpu(); want = want.float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} out of tolerance, max abs err {float(err.max()):.3e}"
    return float(err.max())


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).half()


def _event_us(fn, launches=50, rounds=5):
    for _ in range(200):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(rounds):
        e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / launches * 1e3)
    return best


def test_reference_shape_one_launch():
    """triton_matmul_batch at (1, 512, 768, 3072) in one launch against the oracle and against the
    default two-launch form (one fp16 ulp: the two round the same fp32 sums formed in a different
    order); both times are printed."""
    print("chain (1,512,768,3072)", flush=True)
    a = _rand(1, 512, 768, seed=1); b = _rand(768, 3072, seed=2, scale=0.05)
    d = _rand(3072, 768, seed=3, scale=0.05); bias = _rand(3072, seed=4, scale=0.5)
    ag, bg, dg, biasg = a.cuda(), b.cuda(), d.cuda(), bias.cuda()
    got = fused.triton_matmul_batch(ag, bg, dg, biasg, single_launch=True)
    want = oe.matmul_gelu_matmul(a, b, d, bias)
    err = _close(got, want, "chain vs oracle")
    _close(fused.triton_matmul_batch(ag, bg, dg, biasg), want, "two launches vs oracle")
    W1t, W2t = fused.pack_weight(bg), fused.pack_weight(dg)
    two = fused.gemm_bias_act(fused.gemm_bias_act(ag, W1t, biasg, "gelu_tanh"), W2t, None, "none")
    d2 = float((got.float() - two.float()).abs().max())
    t_chain = _event_us(lambda: fused.gemm_act_gemm(ag, W1t, biasg, W2t, None, "gelu_tanh"))
    t_two = _event_us(lambda: fused.gemm_bias_act(fused.gemm_bias_act(ag, W1t, biasg, "gelu_tanh"), W2t, None, "none"))
    print(f"chain max abs err vs oracle {err:.2e}, vs two launches {d2:.2e}; {t_chain:.1f} us vs {t_two:.1f} us", flush=True)
    ulp = torch.maximum(two.float().abs(), torch.tensor(1.0, device="cuda")) * 2.0 ** -10
    assert bool(((got.float() - two.float()).abs() <= ulp).all())


@pytest.mark.parametrize("act", ["none", "gelu", "gelu_tanh", "relu"])
@pytest.mark.parametrize("M,K,F,H", [(512, 768, 3072, 768), (200, 256, 1024, 256), (1000, 1024, 4096, 1024), (64, 64, 128, 128), (7, 128, 256, 384)])
def test_shapes_activations_and_second_bias(M, K, F, H, act):
    print(f"chain M{M} K{K} F{F} H{H} {act}", flush=True)
    x = _rand(M, K, seed=5); W1 = _rand(K, F, seed=6, scale=0.05); b1 = _rand(F, seed=7, scale=0.5)
    W2 = _rand(F, H, seed=8, scale=0.05); b2 = _rand(H, seed=9, scale=0.5)
    got = fused.gemm_act_gemm(x.cuda(), fused.pack_weight(W1.cuda()), b1.cuda(), fused.pack_weight(W2.cuda()), b2.cuda(), act)
    t = oe.gemm_bias_act(x, W1, b1, act).half().float()          # the intermediate is stored in fp16
    want = t @ W2.float() + b2.float()
    _close(got, want, f"chain {act}")


def test_repeated_calls_leave_the_workspace_clean():
    """Every call must return its workspace to zeros: the same inputs give the same result call
    after call, also after a call of another shape has used the same buffer."""
    x = _rand(300, 768, seed=10).cuda(); W1t = _rand(3072, 768, seed=11, scale=0.05).cuda()
    b1 = _rand(3072, seed=12, scale=0.5).cuda(); W2t = _rand(768, 3072, seed=13, scale=0.05).cuda()
    first = fused.gemm_act_gemm(x, W1t, b1, W2t, None, "gelu").clone()
    small = fused.gemm_act_gemm(x[:70], W1t, b1, W2t, None, "gelu")
    for i in range(5):
        again = fused.gemm_act_gemm(x, W1t, b1, W2t, None, "gelu")
        ulp = torch.maximum(first.float().abs(), torch.tensor(1.0, device="cuda")) * 2.0 ** -10
        assert bool(((again.float() - first.float()).abs() <= ulp).all()), f"call {i} differs from the first"
    assert bool(((small.float() - first[:70].float()).abs() <= ulp[:70]).all())
    torch.cuda.synchronize()
    ws = next(iter(fused._chain_ws.values()))
    assert int(ws.count_nonzero()) == 0


def test_encoder_layer_small_batch_with_chained_ffn():
    """BERT-base layer at B1 S512 (the size the chained form is for) with ffn_chain on and off,
    against the oracle that rounds where the kernels store fp16."""
    cfg = configs.LayerConfig("small", 1, 512, 768, 12, 3072, 1)
    w = configs.layer_weights(cfg.hidden, cfg.ffn, seed=0)
    x = configs.layer_input(cfg, seed=1)
    mask = configs.mask_c1(cfg.seq)[None].float()
    lut = pm.get_sparse_storage(mask.cuda(), 64, 64)[1:]
    wg = {k: v.cuda() for k, v in w.items()}
    want = oe.bert_layer(x, w, mask, cfg.heads, eps=1e-12, gelu="erf", round_fp16="split")
    for chain in (True, False, "auto"):
        got = EncoderLayer(wg, cfg.heads, ffn_chain=chain)(x.cuda(), lut)
        err = _close(got, want, f"layer ffn_chain={chain}")
        print(f"layer B1 S512 ffn_chain={chain}: max abs err {err:.2e}", flush=True)


def test_errors():
    x = _rand(64, 128, seed=14).cuda()
    with pytest.raises(StofError):
        fused.gemm_act_gemm(x, _rand(192, 128).cuda(), None, _rand(128, 192).cuda())       # F % 128
    with pytest.raises(StofError):
        fused.gemm_act_gemm(x, _rand(256, 128).cuda(), None, _rand(64, 256).cuda())        # H % 128
    with pytest.raises(StofError):
        fused.gemm_act_gemm(x, _rand(256, 64).cuda(), None, _rand(128, 256).cuda())        # W1t does not match K
