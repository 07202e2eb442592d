"""GPU parity of the attention kernels on bfloat16 tensors (the reference computes in fp16 only,
src/ops/package_op.py:50-66; this format is an addition behind the same operators), against the
CPU oracle in fp32 on the same bf16-rounded inputs.

Tolerance: bfloat16 keeps 8 significant bits, so the probabilities and the stored result carry a
relative rounding error of 2^-9 each where fp16 carries 2^-12:
    |got - want| <= 8e-3 + 1.6e-2 * |want|
(the fp16 tests' bound with its absolute part times four and its relative part times 1.6;
observed max abs error 6.4e-3, on outputs of magnitude 2 to 4 whose bf16 half-ulp is 7.8e-3).
"""
import pytest
import torch

from oracle import attention as oa
from stof import configs, masks as pm
from stof.ops import block_attn, rowwise_attn, StofError

pytestmark = pytest.mark.gpu
ATOL, RTOL = 8e-3, 1.6e-2
FORMS = ["two_rows", "key_split", "pipelined"]


def _close(got, want, what=""):
    assert got.dtype == torch.bfloat16
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    bad = err > ATOL + RTOL * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements out of tolerance, max abs err {float(err.max()):.3e}"
    print(f"{what}: max abs err {float(err.max()):.3e}", flush=True)


def _inputs(b, h, s, seed, scale=1.0):
    cfg = configs.AttnConfig("t", b, h, s)
    return configs.qkv(cfg, seed=seed, dtype=torch.bfloat16, device="cuda", scale=scale)


def _oracle(q, k, v, mask):
    return oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask.cpu())


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("name,b,h,s", [("C1", 1, 12, 512), ("C2", 8, 12, 1024), ("C5", 2, 4, 2048)])
def test_config_shapes_vs_oracle(name, b, h, s, form):
    print(f"case bf16 {name} b{b} h{h} s{s} {form}", flush=True)
    mask = configs.ATTN_MASKS[name](s)
    q, k, v = _inputs(b, h, s, seed=0)
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    got = block_attn(q, k, v, lut, 64, 64, launch_form=form)
    _close(got, _oracle(q, k, v, mask), f"{name} {form}")


@pytest.mark.parametrize("form", FORMS)
def test_random_mask_with_partial_tiles_and_bshd_output(form):
    print(f"case bf16 random mask {form}", flush=True)
    S = 512
    g = torch.Generator().manual_seed(3)
    mask = torch.rand(S, S, generator=g) < 0.3
    mask[:, 128:192] = False          # an empty key block
    mask[64:128, :64] = True          # a full tile
    mask[200] = False                 # a row without keys: zeros on both sides
    q, k, v = _inputs(2, 4, S, seed=4)
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    got = block_attn(q, k, v, lut, 64, 64, launch_form=form, out_layout="bshd")
    assert got.shape == (2, S, 4 * 64)
    want = _oracle(q, k, v, mask)
    _close(got.view(2, S, 4, 64).permute(0, 2, 1, 3), want, f"random mask {form}")


@pytest.mark.parametrize("form", FORMS)
def test_rising_and_large_logits(form):
    """Scores of several hundred that rise from one key block to the next (every tile raises the
    running max; the pipelined form repeats its walk on the exact path)."""
    print(f"case bf16 rising logits {form}", flush=True)
    B, H, S = 2, 4, 512
    g = torch.Generator().manual_seed(11)
    q = (torch.ones(B, H, S, 64) * 0.5 + 0.05 * torch.randn(B, H, S, 64, generator=g)).bfloat16().cuda()
    ramp = torch.arange(S).float()[None, None, :, None] / S * 12.0
    k = (ramp * torch.ones(B, H, S, 64) + 0.05 * torch.randn(B, H, S, 64, generator=g)).bfloat16().cuda()
    v = torch.randn(B, H, S, 64, generator=g).bfloat16().cuda()
    mask = torch.ones(S, S, dtype=torch.bool)
    mask[70:90, :] &= torch.rand(20, S, generator=g) < 0.5
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    got = block_attn(q, k, v, lut, 64, 64, launch_form=form)
    assert bool(torch.isfinite(got.float()).all())
    _close(got, _oracle(q, k, v, mask), f"rising logits {form}")


@pytest.mark.parametrize("form", FORMS)
def test_rowwise_kinds(form):
    print(f"case bf16 rowwise {form}", flush=True)
    q, k, v = _inputs(2, 4, 512, seed=5)
    qc, kc, vc = (t.cpu().float() for t in (q, k, v))
    for causal in (False, True):
        _close(rowwise_attn("full", q, k, v, causal, launch_form=form),
               oa.rowwise_attn_full(qc, kc, vc, causal), f"full causal={causal} {form}")
    _close(rowwise_attn("sliding", q, k, v, True, 96, launch_form=form),
           oa.rowwise_attn_sliding(qc, kc, vc, True, 96), f"sliding {form}")
    rm = (torch.rand(512, 512, generator=torch.Generator().manual_seed(6)) < 0.4).half()
    rm[:, 0] = 1
    _close(rowwise_attn("mask", q, k, v, False, 0, rm.cuda(), launch_form=form),
           oa.rowwise_attn_mask(qc, kc, vc, False, rm), f"mask {form}")


def test_mixed_formats_raise():
    q, k, v = _inputs(1, 2, 128, seed=7)
    lut = pm.get_sparse_storage(torch.ones(1, 128, 128).cuda(), 64, 64)[1:]
    with pytest.raises(StofError):
        block_attn(q, k.half(), v, lut)
    with pytest.raises(StofError):
        block_attn(q.float(), k.float(), v.float(), lut)
    with pytest.raises(StofError):
        block_attn(q, k, v, lut, out=torch.empty(1, 128, 128, dtype=torch.float16, device="cuda"), out_layout="bshd")
