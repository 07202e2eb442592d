"""GPU parity of the block-masked attention kernel, through the Python operator API and
the C ABI underneath, against the CPU oracle on the same seeded inputs.

Tolerance (fp16 kernel vs fp32 oracle on the same fp16-rounded inputs):
    |got - want| <= 2e-3 + 1e-2 * |want|        (max-abs 2e-3, rel 1e-2)
Rows without any allowed key are defined as zero on both sides.
"""
import numpy as np
import pytest
import torch

from oracle import attention as oa
from oracle import masks as om
from stof import configs, masks as pm
from stof.ops import block_attn, block_attn_mask_op, StofError

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-3, 1e-2


@pytest.fixture(autouse=True, params=["two_rows", "key_split", "pipelined"])
def launch_form(request):
    """Every test of this module runs once per launch form of the kernel."""
    from stof.ops import set_attention_launch_form
    set_attention_launch_form(request.param)
    yield request.param
    set_attention_launch_form("auto")


def _close(got, want, what=""):
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    bad = err > ATOL + RTOL * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements out of tolerance, max abs err {float(err.max()):.3e}"
    return float(err.max())


def _inputs(b, h, s, seed, scale=1.0):
    cfg = configs.AttnConfig("t", b, h, s)
    return configs.qkv(cfg, seed=seed, dtype=torch.float16, device="cuda", scale=scale)


def _run(q, k, v, mask2d, **kw):
    lut = pm.get_sparse_storage(mask2d.float()[None].cuda(), 64, 64)[1:]
    return block_attn(q, k, v, lut, 64, 64, **kw)


def _oracle(q, k, v, mask):
    return oa.dense_masked_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(), mask.cpu())


@pytest.mark.parametrize("name,b,h,s", [("C1", 1, 12, 512), ("C2", 8, 12, 1024), ("C5", 2, 4, 2048)])
def test_config_shapes_vs_oracle(name, b, h, s):
    print(f"case {name} b{b} h{h} s{s}", flush=True)
    mask = configs.ATTN_MASKS[name](s)
    q, k, v = _inputs(b, h, s, seed=0)
    got = _run(q, k, v, mask)
    torch.cuda.synchronize()
    _close(got, _oracle(q, k, v, mask), name)


def test_c4_full_size_subset_and_properties():
    """C4 at its full shape: oracle on a subset of (batch, head) pairs, plus size-independent
    properties on the whole output (rows of ones for V == 1, linearity in V)."""
    print("case C4 full", flush=True)
    cfg = configs.C4
    mask = configs.mask_c4(cfg.seq)
    q, k, v = configs.qkv(cfg, seed=0, device="cuda")
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    assert lut[5][-1].item() == 946
    got = block_attn(q, k, v, lut)
    for (b, h) in [(0, 0), (1, 15), (0, 7)]:
        want = _oracle(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], mask)
        _close(got[b:b + 1, h:h + 1], want, f"C4 b{b} h{h}")
    ones = block_attn(q, k, torch.ones_like(v), lut)
    assert float((ones.float() - 1).abs().max()) <= 2e-3
    v2 = torch.randn_like(v)
    a = block_attn(q, k, v, lut).float(); b2 = block_attn(q, k, v2, lut).float()
    ab = block_attn(q, k, (v.float() + v2.float()).half(), lut).float()
    assert float((ab - (a + b2)).abs().max()) <= 1e-2   # fp16 rounding of v+v2 and of three outputs


def test_in_place_op_returns_q_like_reference():
    mask = configs.mask_c1(512)
    q, k, v = _inputs(1, 12, 512, seed=1)
    want = _oracle(q, k, v, mask)
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)
    ret = block_attn_mask_op(q, k, v, *lut[1:], 64, 64, 4)
    assert ret.data_ptr() == q.data_ptr()
    _close(q, want, "in place")


def test_non_contiguous_q_receives_result():
    mask = configs.mask_c1(256)
    q, k, v = _inputs(1, 4, 256, seed=2)
    want = _oracle(q, k, v, mask)
    qt = q.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)     # [B,H,S,D] view, S/H swapped in memory
    qd = torch.empty(1, 4, 256, 128, dtype=torch.float16, device="cuda")[..., ::2]  # D stride 2
    qd.copy_(q)
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)
    _close(block_attn_mask_op(qt, k, v, *lut[1:], 64, 64, 4), want, "strided q")
    _close(block_attn_mask_op(qd, k, v, *lut[1:], 64, 64, 4), want, "q with D stride 2")


def test_packed_qkv_views_and_bshd_output():
    """q, k, v as slices of one [B,S,3*H*D] projection buffer; output written as [B,S,H*D]."""
    B, H, S, D = 2, 6, 512, 64
    g = torch.Generator().manual_seed(3)
    packed = torch.randn(B, S, 3 * H * D, generator=g).half().cuda()
    q, k, v = (packed[..., t * H * D:(t + 1) * H * D].view(B, S, H, D).permute(0, 2, 1, 3) for t in range(3))
    mask = configs.mask_c5(S)
    out = _run(q, k, v, mask, out_layout="bshd")
    want = _oracle(q, k, v, mask).permute(0, 2, 1, 3).reshape(B, S, H * D)
    assert out.shape == (B, S, H * D)
    _close(out, want, "packed/bshd")


def test_per_sample_lut_padding_mask():
    """C3's mask at reduced batch: one LUT per sample (key padding x sliding window)."""
    B, H, S = 4, 12, 512
    mask, L = configs.mask_c3(batch=B, s=S, window=256, seed=0)
    q, k, v = _inputs(B, H, S, seed=4)
    lut = pm.get_sparse_storage_batched(mask.float().cuda(), 64, 64)[1:]
    got = block_attn(q, k, v, lut)
    _close(got, _oracle(q, k, v, mask), "per-sample LUT")


def test_dead_rows_empty_blocks_and_masked_first_tile():
    S = 256
    mask = torch.ones(S, S)
    mask[64:128, :] = 0                 # a query block with no LUT entry -> zeros
    mask[3, :] = 0                      # a dead row inside a live block
    mask[130, :64] = 0                  # row masked in its FIRST visited (partial) tile only
    mask[131, :] = 0; mask[131, 255] = 1   # single allowed key, in the last tile
    q, k, v = _inputs(2, 3, S, seed=5)
    got = _run(q, k, v, mask)
    assert bool((got[:, :, 64:128] == 0).all()) and bool((got[:, :, 3] == 0).all())
    _close(got, _oracle(q, k, v, mask), "edge rows")
    assert torch.allclose(got[:, :, 131].float(), v[:, :, 255].float(), atol=1e-3)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_block_masks(seed):
    """Random full / partial / empty tiling, random element masks inside partial tiles."""
    rng = np.random.default_rng(seed)
    S = 64 * int(rng.integers(2, 9))
    n = S // 64
    kind = rng.integers(0, 3, size=(n, n))
    mask = torch.zeros(S, S)
    for r in range(n):
        for c in range(n):
            if kind[r, c] == 1:
                mask[r * 64:(r + 1) * 64, c * 64:(c + 1) * 64] = 1
            elif kind[r, c] == 2:
                dens = rng.choice([0.02, 0.5, 0.98])
                mask[r * 64:(r + 1) * 64, c * 64:(c + 1) * 64] = torch.from_numpy(
                    (rng.random((64, 64)) < dens).astype(np.float32))
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    print(f"seed {seed}: S {S} B {B} H {H}", flush=True)
    q, k, v = _inputs(B, H, S, seed=10 + seed)
    got = _run(q, k, v, mask)
    _close(got, _oracle(q, k, v, mask), f"random seed {seed}")
    # the oracle's restatement of the reference's block algorithm agrees as well
    lut_np = om.get_sparse_storage(mask.numpy()[None], 64, 64)
    blk = oa.block_attn_mask(q.cpu().float().numpy(), k.cpu().float().numpy(), v.cpu().float().numpy(), lut_np, 64, 64)
    _close(got, torch.from_numpy(blk), f"random seed {seed} (block oracle)")


@pytest.mark.parametrize("b,h,s,seed", [(2, 4, 1024, 20), (4, 4, 512, 21), (1, 8, 192, 22), (8, 2, 2048, 23)])
def test_length_ordered_placement(b, h, s, seed):
    """Batch x heads a multiple of 8: workgroups take their query blocks in descending order of
    LUT row length (ranked inside the kernel).  Rows of very different and of equal lengths, an
    empty row, an odd block count: every block must still be computed exactly once."""
    rng = np.random.default_rng(seed)
    n = s // 64
    blk = np.zeros((n, n), dtype=bool)
    for r in range(n):
        cnt = int(rng.choice([0, 1, 2, n // 2, n]))        # many ties, some empty, some full rows
        blk[r, rng.choice(n, size=cnt, replace=False)] = True
    mask = torch.from_numpy(np.kron(blk, np.ones((64, 64), dtype=np.float32)))
    holes = torch.from_numpy((rng.random((s, s)) < 0.9).astype(np.float32))
    part = torch.from_numpy(np.kron(rng.random((n, n)) < 0.3, np.ones((64, 64), dtype=np.float32)))
    mask = mask * (1 - part) + mask * part * holes          # a third of the blocks become partial
    print(f"placement b{b} h{h} s{s} rows {blk.sum(1).tolist()}", flush=True)
    q, k, v = _inputs(b, h, s, seed=seed)
    got = _run(q, k, v, mask)
    _close(got, _oracle(q, k, v, mask), "length-ordered placement")
    per_sample = torch.stack([mask if i % 2 == 0 else torch.flip(mask, dims=(0,)) for i in range(b)])
    lut = pm.get_sparse_storage_batched(per_sample.float().cuda(), 64, 64)[1:]
    _close(block_attn(q, k, v, lut), _oracle(q, k, v, per_sample), "length-ordered placement, LUT per sample")


def test_mask_that_allows_nothing_gives_zeros():
    """Every LUT row empty: the column lists have no entries at all (NULL at the C boundary)."""
    for b, h, s in ((1, 2, 64), (2, 4, 256)):
        q, k, v = _inputs(b, h, s, seed=30)
        got = _run(q, k, v, torch.zeros(s, s))
        assert bool((got == 0).all())


@pytest.mark.parametrize("S", [64, 192])
def test_single_and_odd_query_block_counts(S):
    """One query block, and a block count that leaves the last two-row workgroup half empty."""
    g = torch.Generator().manual_seed(S)
    mask = (torch.rand(S, S, generator=g) < 0.6).float()
    mask[:, :64] = 1                                  # a full tile in every row
    q, k, v = _inputs(2, 3, S, seed=8)
    _close(_run(q, k, v, mask), _oracle(q, k, v, mask), f"S {S}")


def test_long_sequence_walks_several_column_windows():
    """S 8192 = 128 key blocks: the kernel walks a LUT row in windows of 64 key blocks, so rows
    here span two windows, with partial tiles in both and rows that skip the first window."""
    S = 8192
    i = torch.arange(S)[:, None]; j = torch.arange(S)[None, :]
    mask = (((i - j) >= 0) & ((i - j) < 300)) | ((j <= i) & ((j // 64) % 37 == 3)) | ((i < 64) & (j >= 4500) & (j < 4700))
    q, k, v = _inputs(1, 2, S, seed=9)
    got = _run(q, k, v, mask.float())
    _close(got, _oracle(q, k, v, mask.float()), "S 8192")
    # 8 heads: whole heads per XCD, so the 64 pairs of query blocks of a head are taken in length
    # order (two rows per workgroup; with the key split 128 rows exceed the limit: plain order)
    q, k, v = _inputs(1, 8, S, seed=10)
    got = _run(q, k, v, mask.float())
    _close(got, _oracle(q, k, v, mask.float()), "S 8192, 8 heads")


def test_large_logits_no_overflow():
    """|score| of several hundred: the max-subtracted softmax must stay finite."""
    q, k, v = _inputs(1, 2, 256, seed=6, scale=6.0)
    mask = configs.mask_c1(256)
    got = _run(q, k, v, mask)
    assert bool(torch.isfinite(got).all())
    _close(got, _oracle(q, k, v, mask), "large logits")


@pytest.mark.parametrize("S", [512, 1024])
def test_rising_logits_along_the_keys(S):
    """Scores that grow by far more than the fp16 range of the probabilities from one key block
    to the next: every tile raises the running max.  (The software-pipelined launch form takes
    the max as it stands on its fast path and verifies the row sums; here the verification
    fails and the workgroup repeats its walk on the exact path.)"""
    B, H = 2, 4
    g = torch.Generator().manual_seed(11)
    q = (torch.ones(B, H, S, 64) * 0.5 + 0.05 * torch.randn(B, H, S, 64, generator=g)).half().cuda()
    ramp = torch.arange(S).float()[None, None, :, None] / S * 12.0           # q.k rises by about 24 per 64 keys
    k = (ramp * torch.ones(B, H, S, 64) + 0.05 * torch.randn(B, H, S, 64, generator=g)).half().cuda()
    v = torch.randn(B, H, S, 64, generator=g).half().cuda()
    mask = torch.ones(S, S, dtype=torch.bool)
    mask[:, S // 2:S // 2 + 64] = False                                        # one empty key block
    mask[70:90, :] &= torch.rand(20, S, generator=g) < 0.5                      # and some partial tiles
    got = _run(q, k, v, mask)
    assert bool(torch.isfinite(got).all())
    _close(got, _oracle(q, k, v, mask), "rising logits")


def test_error_paths_raise():
    q, k, v = _inputs(1, 2, 128, seed=7)
    lut = pm.get_sparse_storage(torch.ones(1, 128, 128).cuda(), 64, 64)[1:]
    with pytest.raises(StofError):
        block_attn(q.float(), k, v, lut)                       # wrong dtype
    with pytest.raises(StofError):
        block_attn(q, k, v, lut, 32, 32)                       # row pointers do not fit 32x32
    lut48 = pm.get_sparse_storage(torch.ones(1, 192, 192).cuda(), 48, 48)[1:]
    q192 = torch.randn(1, 2, 192, 64, device="cuda").half()
    with pytest.raises(StofError):
        block_attn(q192[:, :, :128], q192[:, :, :128], q192[:, :, :128], lut48, 48, 48)   # row pointers do not fit
    bad = list(lut); bad[5] = lut[5].long()
    with pytest.raises(StofError):
        block_attn(q, k, v, tuple(bad))                        # int64 row pointers
    bad = list(lut); bad[6] = torch.flip(lut[6], dims=[0])
    with pytest.raises(StofError):
        block_attn(q, k, v, tuple(bad))                        # column indices not ascending within rows
    bad = list(lut); bad[6] = lut[6] + 5
    with pytest.raises(StofError):
        block_attn(q, k, v, tuple(bad))                        # column index out of range
    q96 = torch.randn(1, 2, 128, 96, device="cuda").half()
    with pytest.raises(StofError):
        block_attn(q96, q96, q96, lut)                         # head size 96


def _unpack_bits(words, cols):
    """int64 bit rows [rows, cols/64] -> bool [rows, cols] (bit t of word w = column 64w + t)."""
    w = words.cpu().numpy().view(np.uint64)
    t = np.arange(64, dtype=np.uint64)
    return ((w[:, :, None] >> t[None, None, :]) & np.uint64(1)).astype(bool).reshape(w.shape[0], cols)


@pytest.mark.parametrize("additive", [True, False])
def test_pack_mask_bits_vector_and_scalar_paths(additive):
    """Bit-exact against numpy; the 16-byte path (contiguous rows) and the scalar path (row
    pitch not a multiple of 8 elements, reached through the C ABI) must agree."""
    from stof import _lib
    from stof.ops import pack_mask_bits
    g = torch.Generator().manual_seed(5)
    rows, cols = 200, 192          # 600 words: not a multiple of the 8 words a wavefront packs per pass
    keep = torch.rand(rows, cols, generator=g) < 0.4
    src = torch.where(keep, 0.0, -10000.0) if additive else keep.float()
    src = src.half().cuda()
    got = pack_mask_bits(src, additive=additive)
    assert np.array_equal(_unpack_bits(got, cols), keep.numpy())
    # scalar path: rows at a pitch of cols + 4 elements
    ld = cols + 4
    padded = torch.zeros(rows, ld, dtype=torch.float16, device="cuda")
    padded[:, :cols] = src
    dst = torch.zeros(rows, cols // 64, dtype=torch.int64, device="cuda")
    rc = _lib.lib().stof_pack_mask_bits(padded.data_ptr(), dst.data_ptr(), rows, cols, ld, 1 if additive else 0, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert np.array_equal(_unpack_bits(dst, cols), keep.numpy())


@pytest.mark.parametrize("mask", ["causal", "bigbird", "sliding"])
def test_example_script_runs(mask):
    """The example that follows the reference's unified attention benchmark, end to end."""
    import subprocess, sys, os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = os.path.join(root, "sc25-stof-ad_amd", "examples", "unified_attention.py")
    r = subprocess.run([sys.executable, script, "--mask", mask, "--batch", "2", "--heads", "4", "--seq", "512", "--iters", "5"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [l for l in r.stdout.splitlines() if l.startswith("max abs difference")][0]
    assert float(line.split(":")[1]) < 5e-3, r.stdout


def test_bound_attention_on_fixed_buffers():
    """BoundAttention: arguments resolved once, then launches on new contents of the same tensors give
    what block_attn gives (bit for bit: the same kernel on the same arguments), in both output layouts."""
    from stof.ops import BoundAttention
    B, H, S = 2, 3, 512
    mask = configs.mask_c1(S)
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    q, k, v = _inputs(B, H, S, seed=21)
    for layout in ("bhsd", "bshd"):
        out = torch.empty((B, H, S, 64) if layout == "bhsd" else (B, S, H * 64), dtype=torch.float16, device="cuda")
        run = BoundAttention(q, k, v, lut, out=out, out_layout=layout)
        assert run.out is out
        assert torch.equal(out, block_attn(q, k, v, lut, out_layout=layout))           # the constructor's launch
        q2, k2, v2 = _inputs(B, H, S, seed=22)
        q.copy_(q2); k.copy_(k2); v.copy_(v2)                                           # new contents, same buffers
        got = run()
        assert got is out
        assert torch.equal(out, block_attn(q2, k2, v2, lut, out_layout=layout))
    _close(block_attn(q, k, v, lut), _oracle(q, k, v, mask), "bound attention inputs")
