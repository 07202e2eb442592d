"""The precomputed walk ("plan") of a LUT: its contents against a host restatement of the merged
walk (integer-exact), and attention through it against attention without it (bit-identical) and
against the CPU oracle, for shared and per-sample LUTs, both plan group sizes and both formats.

Tolerance vs the fp32 oracle: |got - want| <= 2e-3 + 1e-2 * |want| (fp16)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import attention as oa
from stof import _lib, configs, masks as pm
from stof.ops import block_attn

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-3, 1e-2


def _lut(mask2d):
    return pm.get_sparse_storage(mask2d.float()[None].cuda(), 64, 64)[1:]


def _expected_plan(lut, S, rows):
    """The plan layout restated on the host: per group (ROWS adjacent LUT rows) the ascending
    union of the rows' LOAD lists; groups stored in descending order of walk length."""
    frp, fci, prp, pci, pbm, lrp, lci = [t.cpu().numpy() for t in lut]
    nq = nk = S // 64
    n_groups = (nq + rows - 1) // rows
    stride = (nk + 2 + 7) & ~7
    walks = []
    for g in range(n_groups):
        cols = {}
        p0 = [0, 0]
        for r in range(rows):
            qr = rows * g + r
            if qr >= nq:
                continue
            p0[r] = int(prp[qr])
            part = {int(c): i for i, c in enumerate(pci[prp[qr]:prp[qr + 1]])}
            for c in lci[lrp[qr]:lrp[qr + 1]]:
                w = cols.setdefault(int(c), int(c))
                w |= 1 << (16 + r)
                if int(c) in part:
                    w |= (1 << (18 + r)) | (part[int(c)] << (32 + 16 * r))
                cols[int(c)] = w
        walks.append((g, p0, [cols[c] for c in sorted(cols)]))
    order = sorted(range(n_groups), key=lambda g: (-len(walks[g][2]), g)) if n_groups <= 64 else list(range(n_groups))
    plan = np.zeros((n_groups, stride), dtype=np.uint64)
    for slot, g in enumerate(order):
        _, p0, steps = walks[g]
        plan[slot, 0] = g | (len(steps) << 16)
        plan[slot, 1] = (p0[0] & 0xFFFFFFFF) | ((p0[1] & 0xFFFFFFFF) << 32)
        plan[slot, 2:2 + len(steps)] = np.array(steps, dtype=np.uint64)
    return plan


def _build_plan(lut, S, rows, batches=1, lut_bs=0):
    lib = _lib.lib()
    nbytes = lib.stof_attn_plan_bytes(S, rows, batches)
    assert nbytes > 0
    plan = torch.zeros(nbytes // 8, dtype=torch.int64, device="cuda")
    frp, fci, prp, pci, pbm, lrp, lci = lut
    ptr = lambda t: t.data_ptr() if t.numel() else None
    rc = lib.stof_attn_plan_build(ptr(prp), ptr(pci), ptr(lrp), ptr(lci), S, lut_bs, batches, rows, plan.data_ptr(), nbytes, None)
    assert rc == 0
    torch.cuda.synchronize()
    return plan


@pytest.mark.parametrize("rows", [1, 2])
@pytest.mark.parametrize("name,S", [("C1", 512), ("C4", 4096), ("C5", 2048), ("C2", 1024), ("C1", 192)])
def test_plan_contents_match_host_restatement(name, S, rows):
    print(f"case plan contents {name} S{S} rows{rows}", flush=True)
    lut = _lut(configs.ATTN_MASKS[name](S))
    plan = _build_plan(lut, S, rows)
    want = _expected_plan(lut, S, rows)
    got = plan.cpu().numpy().view(np.uint64).reshape(want.shape)
    n_steps = (want[:, 0] >> np.uint64(16)).astype(np.int64)
    for slot in range(want.shape[0]):                # words past a group's last step are not written
        assert np.array_equal(got[slot, :2 + n_steps[slot]], want[slot, :2 + n_steps[slot]]), f"slot {slot}"


def _rand_block_mask(S, seed, p_full=0.25, p_part=0.15):
    g = torch.Generator().manual_seed(seed)
    n = S // 64
    kind = torch.rand(n, n, generator=g)
    mask = (kind < p_full).repeat_interleave(64, 0).repeat_interleave(64, 1)
    ragged = torch.rand(S, S, generator=g) < 0.5
    part = ((kind >= p_full) & (kind < p_full + p_part)).repeat_interleave(64, 0).repeat_interleave(64, 1)
    return mask | (part & ragged)


@pytest.mark.parametrize("form", ["two_rows", "key_split"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_with_plan_equals_attention_without(form, dtype):
    cases = [("C1", configs.AttnConfig("a", 1, 12, 512), configs.mask_c1(512)),
             ("C5", configs.AttnConfig("b", 2, 4, 2048), configs.mask_c5(2048)),
             ("C4", configs.AttnConfig("c", 1, 4, 4096), configs.mask_c4(4096)),
             ("random blocks", configs.AttnConfig("d", 2, 3, 1024), _rand_block_mask(1024, 5)),
             ("two windows of plan words", configs.AttnConfig("e", 1, 2, 8320), _rand_block_mask(8320, 7, 0.4, 0.1)),
             ("odd block count", configs.AttnConfig("f", 1, 3, 192), torch.ones(192, 192, dtype=torch.bool).tril()),
             ("nothing allowed", configs.AttnConfig("g", 1, 2, 256), torch.zeros(256, 256, dtype=torch.bool))]
    for what, cfg, mask in cases:
        print(f"case plan vs no plan: {what} {form} {dtype}", flush=True)
        q, k, v = configs.qkv(cfg, seed=3, dtype=dtype, device="cuda")
        lut = _lut(mask)
        a = block_attn(q, k, v, lut, launch_form=form, use_plan=True)
        b = block_attn(q, k, v, lut, launch_form=form, use_plan=False)
        torch.cuda.synchronize()
        assert torch.equal(a, b), what
        if dtype == torch.float16 and cfg.seq <= 2048:
            want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask)
            err = (a.float().cpu() - want).abs()
            assert not bool((err > ATOL + RTOL * want.abs()).any()), f"{what}: max err {float(err.max()):.2e}"


def test_per_sample_lut_with_plan():
    """Key-padding masks: one LUT and one plan section per sample."""
    B, H, S = 4, 3, 512
    lens = [512, 300, 129, 64]
    masks = torch.stack([(torch.arange(S)[None, :] < L) & ((torch.arange(S)[:, None] - torch.arange(S)[None, :]).abs() <= 200)
                         for L in lens])
    lut = pm.get_sparse_storage_batched(masks.float().cuda(), 64, 64)[1:]
    q, k, v = configs.qkv(configs.AttnConfig("p", B, H, S), seed=9, device="cuda")
    for form in ("two_rows", "key_split"):
        a = block_attn(q, k, v, lut, launch_form=form, use_plan=True)
        b = block_attn(q, k, v, lut, launch_form=form, use_plan=False)
        assert torch.equal(a, b), form
    for bi, L in enumerate(lens):
        want = oa.dense_masked_attention(q[bi:bi + 1].cpu().float(), k[bi:bi + 1].cpu().float(), v[bi:bi + 1].cpu().float(), masks[bi])
        err = (a[bi:bi + 1, :, :L].float().cpu() - want[:, :, :L]).abs()
        assert not bool((err > ATOL + RTOL * want[:, :, :L].abs()).any()), f"sample {bi}"


def test_planned_entry_point_through_the_c_abi():
    """stof_block_attn_fwd_planned called directly: a plan of the right group size is used, one of
    the other size or NULL is ignored, a short buffer is rejected; all give the same bits."""
    lib = _lib.lib()
    B, H, S = 2, 4, 1024
    mask = _rand_block_mask(S, 21)
    q, k, v = configs.qkv(configs.AttnConfig("x", B, H, S), seed=2, device="cuda")
    lut = _lut(mask)
    frp, fci, prp, pci, pbm, lrp, lci = lut
    from stof.ops import pack_mask_bits
    bits = pack_mask_bits(pbm, additive=True)
    st = _lib.i64x3(H * S * 64, S * 64, 64)
    rows = lib.stof_attn_plan_rows(B, H, S, 0)
    assert rows == 2 and lib.stof_attn_plan_rows(B, H, S, 1) == 1 and lib.stof_attn_plan_rows(B, H, S, 2) == 0
    plans = {r: _build_plan(lut, S, r) for r in (1, 2)}

    def run(plan, plan_rows, nbytes=None, form=0):
        out = torch.empty_like(q)
        rc = lib.stof_block_attn_fwd_planned(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), frp.data_ptr(), fci.data_ptr(), prp.data_ptr(),
            pci.data_ptr(), bits.data_ptr(), lrp.data_ptr(), lci.data_ptr(), 64, 64, 0.125, st, st, st, st,
            B, S, H, 64, 0, 0, form, plan.data_ptr() if plan is not None else None,
            (plan.numel() * 8 if plan is not None else 0) if nbytes is None else nbytes, plan_rows, None)
        torch.cuda.synchronize()
        return rc, out

    rc0, base = run(None, 0)
    assert rc0 == 0
    for form in (0, 1):
        rc_ref, ref = run(None, 0, form=form)
        for r in (1, 2):
            rc, out = run(plans[r], r, form=form)
            assert rc == 0 and torch.equal(out, ref), (form, r)
    rc, _ = run(plans[2], 2, nbytes=64)
    assert rc == -2
    want = oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask)
    err = (base.float().cpu() - want).abs()
    assert not bool((err > ATOL + RTOL * want.abs()).any())


def _hand_lut(S, device="cuda"):
    """A LUT written down directly (no dense S x S mask, which at these lengths would not fit): query
    block r lists key block 0 (full; for r = 0 it is the diagonal), r - 1 (full) and r (partial: causal
    inside the block)."""
    nq = S // 64
    lci, fci, pci, lrp, frp, prp = [], [], [], [0], [0], [0]
    for r in range(nq):
        full = sorted({0, r - 1} - {r, -1})
        fci += full; pci.append(r); lci += sorted(full + [r])
        frp.append(len(fci)); prp.append(len(pci)); lrp.append(len(lci))
    t = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    tri = torch.tril(torch.ones(64, 64))
    pbm = (-10000.0 * (1 - tri)).half().to(device).expand(nq, 64, 64).contiguous()
    return (t(frp), t(fci), t(prp), t(pci), pbm, t(lrp), t(lci))


@pytest.mark.parametrize("S,planned", [(65536, True), (65600, False)])
def test_longest_sequence_with_a_plan_and_the_first_without(S, planned):
    """1024 key blocks is the longest walk a plan holds; beyond it the operator runs the in-kernel
    walk.  Both against dense attention on a few query blocks (first, second, one in the middle,
    the last), and at the limit the two paths bit for bit."""
    print(f"plan limit S{S}", flush=True)
    lib = _lib.lib()
    assert (lib.stof_attn_plan_bytes(S, 2, 1) > 0) == planned
    g = torch.Generator(device="cuda").manual_seed(S)
    q, k, v = (torch.randn(1, 1, S, 64, device="cuda", generator=g).half() for _ in range(3))
    lut = _hand_lut(S)
    got = block_attn(q, k, v, lut)
    if planned:
        assert torch.equal(got, block_attn(q, k, v, lut, use_plan=False))
    nq = S // 64
    for r in (0, 1, nq // 2 + 1, nq - 1):
        cols = sorted({0, r - 1, r} - {-1})
        keys = torch.cat([torch.arange(64 * c, 64 * c + 64) for c in cols]).cuda()
        qi = torch.arange(64 * r, 64 * r + 64).cuda()
        allow = torch.ones(64, len(keys), dtype=torch.bool, device="cuda")
        allow[:, -64:] = torch.tril(torch.ones(64, 64, dtype=torch.bool, device="cuda"))      # the diagonal block comes last
        s = (q[0, 0, qi].float() @ k[0, 0, keys].float().t()) * 0.125
        s = s.masked_fill(~allow, float("-inf"))
        want = torch.softmax(s, -1) @ v[0, 0, keys].float()
        err = (got[0, 0, qi].float() - want).abs()
        assert bool((err <= ATOL + RTOL * want.abs()).all()), f"S{S} query block {r}: max err {float(err.max()):.2e}"
