"""The operator / launch-form selector followed end to end on the GPU (reference:
select_operator and its use, src/benchmk_attn_unified.py:100-163): for every workload
``select_operator`` -> ``apply`` -> the chosen operator in the chosen launch form, result
against the CPU oracle at |got - want| <= 2e-3 + 1e-2 |want|, and the chosen launch form timed
against the other one (HIP events, the launch form passed per call; the times are printed, and
only a gross mis-selection - half again as slow - fails the test)."""
import pytest
import torch

from oracle import attention as oa
from stof import configs, masks as pm, selector
from stof.ops import block_attn, rowwise_attn

pytestmark = pytest.mark.gpu


def _close(got, want, what):
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    bad = err > 2e-3 + 1e-2 * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} out of tolerance, max abs err {float(err.max()):.3e}"


def _event_ms(fn, launches=40, rounds=5):
    """Best of `rounds` event-timed batches of `launches` calls, after a warm-up long enough for
    the clocks to settle."""
    for _ in range(300):
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
        best = min(best, e0.elapsed_time(e1) / launches)
    return best


CASES = [
    # name, B, H, S, mask, causal predicate?, (batch, head) pairs checked against the oracle (None: all)
    ("C1", 1, 12, 512, configs.mask_c1, False, None),
    ("C2", 8, 12, 1024, configs.mask_c2, False, [(0, 0), (7, 11), (3, 5)]),
    ("C2/B4", 4, 12, 1024, configs.mask_c2, False, [(0, 0), (3, 11)]),
    ("C4", 2, 16, 4096, configs.mask_c4, False, [(0, 0), (1, 15)]),
    ("C5-attention", 4, 16, 2048, configs.mask_c5, False, [(0, 3), (3, 12)]),
    ("dense", 2, 12, 1024, lambda s: torch.ones(s, s, dtype=torch.bool), False, [(0, 0), (1, 11)]),
    ("causal", 2, 12, 2048, lambda s: torch.tril(torch.ones(s, s)).bool(), True, [(0, 0), (1, 7)]),
]


@pytest.mark.parametrize("name,B,H,S,mask_fn,causal,pairs", CASES, ids=[c[0] for c in CASES])
def test_selected_operator_and_form(name, B, H, S, mask_fn, causal, pairs):
    print(f"selector case {name}", flush=True)
    mask = mask_fn(S)
    q, k, v = configs.qkv(configs.AttnConfig(name, B, H, S), seed=0, device="cuda")
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    sel = selector.select_operator(selector.GPUParams(), lut[5], B, S, H, is_causal=causal, lut=lut)
    assert sel.operator == ("row-wise" if name in ("dense", "causal") else "block-wise"), str(sel)
    got = selector.apply(sel, q, k, v, lut, is_causal=causal)               # [B,S,H*D]
    assert got.shape == (B, S, H * 64)
    got = got.view(B, S, H, 64).permute(0, 2, 1, 3)
    for (b, h) in (pairs or [(b, h) for b in range(B) for h in range(H)]):
        want = oa.dense_masked_attention(q[b:b + 1, h:h + 1].cpu().float(), k[b:b + 1, h:h + 1].cpu().float(),
                                         v[b:b + 1, h:h + 1].cpu().float(), mask)
        _close(got[b:b + 1, h:h + 1], want, f"{name} b{b} h{h} ({sel})")

    # the chosen launch form against the other one, both passed per call
    other = "key_split" if sel.launch_form == "two_rows" else "two_rows"
    out = torch.empty(B, S, H * 64, dtype=torch.float16, device="cuda")
    if sel.operator == "row-wise":
        run = lambda form: (lambda: rowwise_attn("full", q, k, v, causal, launch_form=form))
    else:
        run = lambda form: (lambda: block_attn(q, k, v, lut, out=out, out_layout="bshd", launch_form=form))
    t_sel, t_other = _event_ms(run(sel.launch_form)), _event_ms(run(other))
    print(f"{name}: {sel.launch_form} {t_sel * 1e3:.1f} us, {other} {t_other * 1e3:.1f} us", flush=True)
    # The figures are printed for the record (the rule aims at the faster form within 5 %; bench.py
    # reports the forms side by side).  A parity suite must not turn red on a timing flake, so only
    # a gross mis-selection fails: the chosen form more than half again as slow as the other.
    assert t_sel <= 1.5 * t_other, f"{name}: selected {sel.launch_form} {t_sel * 1e3:.1f} us vs {other} {t_other * 1e3:.1f} us"


def test_per_call_form_overrides_module_default():
    """A call that names its launch form is not affected by the module's default, and both
    forms agree with each other within rounding."""
    from stof.ops import set_attention_launch_form
    mask = configs.mask_c1(512)
    q, k, v = configs.qkv(configs.AttnConfig("t", 1, 12, 512), seed=3, device="cuda")
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask)
    try:
        set_attention_launch_form("two_rows")
        a = block_attn(q, k, v, lut, launch_form="key_split")
        b = block_attn(q, k, v, lut)                      # the default: two_rows now
        c = block_attn(q, k, v, lut, launch_form="two_rows")
    finally:
        set_attention_launch_form("auto")
    assert torch.equal(b, c)
    _close(a, want, "key_split per call"); _close(b, want, "default")
    with pytest.raises(Exception):
        block_attn(q, k, v, lut, launch_form="three_rows")


def test_row_wise_variants_selected_by_mask_kind():
    """select -> apply for the sliding-window and element-mask row-wise operators, result vs the oracle."""
    B, H, S, bw = 2, 4, 1024, 200
    q, k, v = configs.qkv(configs.AttnConfig("rw", B, H, S), seed=4, device="cuda")
    i = torch.arange(S)
    win = (i[:, None] - i[None, :] < bw) & (i[None, :] <= i[:, None])
    lut = pm.get_sparse_storage(win.float()[None].cuda(), 64, 64)[1:]
    sel = selector.select_operator(selector.GPUParams(), lut[5], B, S, H, is_causal=True, lut=lut, mask_kind="sliding", bandwidth=bw)
    assert (sel.operator, sel.row_kind) == ("row-wise", "sliding")
    got = selector.apply(sel, q, k, v, is_causal=True).view(B, S, H, 64).permute(0, 2, 1, 3)
    _close(got, oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), win), "row-wise sliding")
    blk = selector.apply(selector.select_operator(selector.GPUParams(), lut[5], B, S, H, is_causal=True, lut=lut), q, k, v, lut, is_causal=True)
    _close(blk.view(B, S, H, 64).permute(0, 2, 1, 3), oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), win), "block-wise on the same mask")
    g = torch.Generator().manual_seed(8)
    em = torch.rand(S, S, generator=g) < 0.7
    em[:, 0] = True
    sel = selector.select_operator(selector.GPUParams(), None, B, S, H, mask_kind="element")
    assert (sel.operator, sel.row_kind) == ("row-wise", "mask")
    got = selector.apply(sel, q, k, v, row_mask=em.half().cuda()).view(B, S, H, 64).permute(0, 2, 1, 3)
    _close(got, oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), em), "row-wise element mask")
