"""Host logic of the operator / launch-form selector (reference: select_operator,
src/benchmk_attn_unified.py:100-163).  The rule is fixed, so the expected answers are derived by
hand from the workload sizes: two-row workgroups = ceil(S/128) * B * H over 256 compute units."""
import pytest
import torch

from stof import configs, masks as pm, selector


def _lut(mask2d):
    return pm.get_sparse_storage(mask2d.float()[None], 64, 64)


@pytest.mark.parametrize("name,cfg,mask_fn,form,groups", [
    ("C1", configs.AttnConfig("C1", 1, 12, 512), configs.mask_c1, "key_split", 48),     # 0.19 per CU, 8 query blocks
    ("C2", configs.C2, configs.mask_c2, "two_rows", 768),                                # 3.0 per CU: the split would need two rounds
    ("C2/B4", configs.AttnConfig("C2b4", 4, 12, 1024), configs.mask_c2, "key_split", 384),  # 1.5 per CU, 16 query blocks
    ("C4", configs.C4, configs.mask_c4, "two_rows", 1024),                               # 4.0 per CU
    ("C5", configs.AttnConfig("C5", 4, 16, 2048), configs.mask_c5, "two_rows", 1024),
])
def test_launch_form_of_baseline_workloads(name, cfg, mask_fn, form, groups):
    lut = _lut(mask_fn(cfg.seq))
    sel = selector.select_operator(selector.GPUParams(), lut[6], cfg.batch, cfg.seq, cfg.heads)
    assert sel.operator == "block-wise"
    assert sel.launch_form == form
    assert sel.groups_per_cu == pytest.approx(groups / 256)
    full, part = configs.BLOCK_COUNTS[name.split("/")[0]]
    assert sel.rho == pytest.approx((full + part) / (cfg.seq // 64) ** 2)
    assert str(sel) == f"block-wise {form} m64n64"


def test_dense_and_causal_masks_go_row_wise():
    gpu = selector.GPUParams()
    s = 512
    dense = torch.ones(s, s)
    assert str(selector.select_operator(gpu, _lut(dense)[6], 2, s, 12)) == "row-wise"
    causal = torch.tril(torch.ones(s, s))
    # 36 of 64 tiles: sparse against the square, dense against the triangle the causal predicate visits
    assert selector.select_operator(gpu, _lut(causal)[6], 2, s, 12).operator == "block-wise"
    assert selector.select_operator(gpu, _lut(causal)[6], 2, s, 12, is_causal=True).operator == "row-wise"
    # a banded causal mask stays block-wise either way
    band = configs.mask_c5(2048)
    assert selector.select_operator(gpu, _lut(band)[6], 1, 2048, 4, is_causal=True).operator == "block-wise"


def test_row_wise_only_for_exactly_dense_or_causal_luts():
    """With the PART row pointers the answer is exact: a nearly dense mask that still has
    partial tiles must stay on the LUT (the dense row-wise operator would ignore them)."""
    gpu = selector.GPUParams()
    s = 512
    dense = torch.ones(s, s)
    lut = _lut(dense)
    assert selector.select_operator(gpu, lut[6], 2, s, 12, lut=lut[1:]).operator == "row-wise"
    holes = dense.clone(); holes[5, 70] = 0; holes[300, 301] = 0          # 62 full + 2 partial of 64 tiles: rho = 1.0
    lut = _lut(holes)
    assert selector.select_operator(gpu, lut[6], 2, s, 12).operator == "row-wise"                       # density estimate alone
    assert selector.select_operator(gpu, lut[6], 2, s, 12, lut=lut[1:]).operator == "block-wise"
    causal = torch.tril(torch.ones(s, s))
    lut = _lut(causal)
    assert selector.select_operator(gpu, lut[6], 2, s, 12, is_causal=True, lut=lut[1:]).operator == "row-wise"
    assert selector.select_operator(gpu, lut[6], 2, s, 12, is_causal=False, lut=lut[1:]).operator == "block-wise"
    shifted = torch.tril(torch.ones(s, s), diagonal=-1)                   # same tiles listed, different diagonal content
    shifted[0, 0] = 1
    lut = _lut(shifted)
    assert selector.select_operator(gpu, lut[6], 2, s, 12, is_causal=True, lut=lut[1:]).operator == "block-wise"
    assert selector.select_operator(gpu, lut[6], 2, s, 12, is_causal=True).operator == "row-wise"      # the density estimate alone cannot tell


def test_per_sample_row_pointers_and_errors():
    mask, _ = configs.mask_c3(4, 512, 256, seed=0)
    lut = pm.get_sparse_storage_batched(mask.float(), 64, 64)
    sel = selector.select_operator(selector.GPUParams(), lut[6], 4, 512, 12)
    assert sel.operator in ("block-wise", "row-wise") and sel.launch_form == "key_split"   # 192 groups, 8 query blocks
    short = selector.select_operator(selector.GPUParams(), lut[6][:, :3], 4, 128, 12)        # two query blocks: never split
    assert short.launch_form == "two_rows"
    with pytest.raises(ValueError):
        selector.select_operator(selector.GPUParams(), lut[6], 4, 500, 12)
    with pytest.raises(ValueError):
        selector.GPUParams("A100")


def test_stated_mask_kinds_select_the_row_wise_variants():
    """The caller's knowledge of the mask (the reference's benchmark selects its row-wise operator
    by the mask's name, src/benchmk_attn_unified.py:396-407)."""
    gpu = selector.GPUParams()
    s, bw = 1024, 200
    i = torch.arange(s)
    win = ((i[:, None] - i[None, :] < bw) & (i[None, :] <= i[:, None])).float()      # causal sliding window
    lut = _lut(win)
    sel = selector.select_operator(gpu, lut[6], 2, s, 12, is_causal=True, mask_kind="sliding", bandwidth=bw)
    assert (sel.operator, sel.row_kind, sel.bandwidth) == ("row-wise", "sliding", bw)
    # a LUT that lists other tiles than the stated window stays block-wise
    assert selector.select_operator(gpu, _lut(configs.mask_c5(s))[6], 2, s, 12, is_causal=True,
                                    mask_kind="sliding", bandwidth=bw).operator == "block-wise"
    # no LUT at hand: row-wise by the stated kind
    for kind, want in (("dense", "full"), ("causal", "full"), ("sliding", "sliding"), ("element", "mask")):
        sel = selector.select_operator(gpu, None, 2, s, 12, mask_kind=kind, bandwidth=bw)
        assert sel.operator == "row-wise" and sel.row_kind == want and str(sel) == "row-wise"
    with pytest.raises(ValueError):
        selector.select_operator(gpu, None, 2, s, 12)
    with pytest.raises(ValueError):
        selector.select_operator(gpu, None, 2, s, 12, mask_kind="sliding")
    with pytest.raises(ValueError):
        selector.select_operator(gpu, lut[6], 2, s, 12, mask_kind="banded")
