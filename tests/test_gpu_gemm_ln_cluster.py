"""GPU parity of the row-block-cluster form of GEMM + bias + residual + LayerNorm against the
CPU oracle.  Tolerance: |got - want| <= 2e-3 + 1e-2 * |want|."""
import pytest
import torch

from oracle import encoder as oe
from stof import fused

pytestmark = pytest.mark.gpu


def _close(got, want, what="", atol=2e-3, rtol=1e-2):
    got = got.float().cpu(); want = want.float().cpu()
    assert got.shape == want.shape
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} out of tolerance, max abs err {float(err.max()):.3e}"


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).half()


# (8192, 768, 768) / (8192, 768, 3072) / (8192, 1024, 4096): the encoder shapes (one resident round);
# (1000, 1024, 1024): ragged last row block; (7, 256, 64): a single partly filled cluster;
# (40000, 512, 128): more tiles than workgroups (each workgroup walks over several tiles);
# eps 1e-12 with a row offset of 30: statistics that a one-pass variance would lose
# (3000, 384, 192) / (5000, 640, 128) / (2050, 896, 64): the odd cluster sizes (3, 5, 7 workgroups per row block)
@pytest.mark.parametrize("M,N,K", [(8192, 768, 768), (8192, 768, 3072), (8192, 1024, 4096), (1000, 1024, 1024),
                                   (7, 256, 64), (40000, 512, 128), (3000, 384, 192), (5000, 640, 128), (2050, 896, 64)])
@pytest.mark.parametrize("eps", [1e-5, 1e-12])
def test_gemm_ln_cluster_matches_oracle(M, N, K, eps):
    print(f"gemm_ln cluster M{M} N{N} K{K} eps{eps}", flush=True)
    x = _rand(M, K, seed=6); W = _rand(K, N, seed=7, scale=0.05); b = _rand(N, seed=8, scale=0.5)
    r = _rand(M, N, seed=9); gm = (1 + 0.1 * _rand(N, seed=10).float()).half(); bt = _rand(N, seed=11, scale=0.1)
    if eps == 1e-12:
        r = (r.float() + 30.0).half()
    args = (x.cuda(), fused.pack_weight(W.cuda()), b.cuda(), r.cuda(), gm.cuda(), bt.cuda(), eps)
    got = fused.gemm_bias_residual_layernorm(*args, form="cluster")
    assert not fused.cluster_exchange_failed()
    _close(got, oe.gemm_bias_residual_layernorm(x, W, b, r, gm, bt, eps), "cluster")
    # a second call on the same workspace (its counters must be back at zero), equal bit for bit
    again = fused.gemm_bias_residual_layernorm(*args, form="cluster")
    assert not fused.cluster_exchange_failed()
    assert torch.equal(got, again)


def test_gemm_ln_cluster_many_tiles_long_k_repeated():
    """Eight times more tiles than the chip holds workgroups, a long K loop, forty launches: no
    wait may run out (a workgroup only waits for workgroups that are running) and every launch
    gives the bits of the first, which agrees with the tiled GEMM followed by the LayerNorm
    kernel within the fp16 rounding of that path's intermediate."""
    M, N, K = 32768, 1024, 2048
    x = _rand(M, K, seed=50).cuda(); Wt = fused.pack_weight(_rand(K, N, seed=51, scale=0.05).cuda())
    b = _rand(N, seed=52, scale=0.5).cuda(); r = _rand(M, N, seed=53).cuda()
    gm = (1 + 0.1 * _rand(N, seed=54).float()).half().cuda(); bt = _rand(N, seed=55, scale=0.1).cuda()
    first = fused.gemm_bias_residual_layernorm(x, Wt, b, r, gm, bt, 1e-5, form="cluster").clone()
    _close(first, fused.gemm_bias_residual_layernorm(x, Wt, b, r, gm, bt, 1e-5, form="split"), "cluster vs split", atol=6e-3)
    out = torch.empty_like(first)
    for i in range(40):
        fused.gemm_bias_residual_layernorm(x, Wt, b, r, gm, bt, 1e-5, out=out, form="cluster")
        if i % 8 == 7:
            assert torch.equal(out, first), f"launch {i} differs"
    assert not fused.cluster_exchange_failed()


def test_gemm_ln_cluster_optional_operands_and_errors():
    x = _rand(300, 128, seed=1); W = _rand(128, 256, seed=2, scale=0.1)
    got = fused.gemm_bias_residual_layernorm(x.cuda(), fused.pack_weight(W.cuda()), None, None, None, None, 1e-5, form="cluster")
    zero_n, one_n = torch.zeros(256).half(), torch.ones(256).half()
    _close(got, oe.gemm_bias_residual_layernorm(x, W, zero_n, torch.zeros(300, 256).half(), one_n, zero_n, 1e-5), "no optional operands")
    with pytest.raises(fused.StofError):
        fused.gemm_bias_residual_layernorm(x.cuda()[:, :96].contiguous(), fused.pack_weight(W.cuda()[:96]), None, None, None, None,
                                           1e-5, form="cluster")   # K % 64 != 0
    Wbad = _rand(128, 320, seed=3)
    with pytest.raises(fused.StofError):
        fused.gemm_bias_residual_layernorm(x.cuda(), fused.pack_weight(Wbad.cuda()), None, None, None, None, 1e-5, form="cluster")


def test_gemm_ln_cluster_in_a_captured_graph():
    """The cluster form recorded into a HIP graph (workspace allocated and zero-filled by torch
    inside the capture): every replay, with eager launches and synchronisation between the
    replays, reproduces the eager result bit for bit."""
    M, N, K = 4096, 768, 768
    xs = [_rand(M, K, seed=20 + i).cuda() for i in range(3)]
    W = fused.pack_weight(_rand(K, N, seed=30, scale=0.05).cuda()); b = _rand(N, seed=31, scale=0.5).cuda()
    r = _rand(M, N, seed=32).cuda(); gm = (1 + 0.1 * _rand(N, seed=33).float()).half().cuda(); bt = _rand(N, seed=34, scale=0.1).cuda()
    run = lambda x: fused.gemm_bias_residual_layernorm(x, W, b, r, gm, bt, 1e-12, form="cluster")
    xin = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(xin)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = run(xin)
    for i, x in enumerate(xs):
        print(f"graph replay {i}", flush=True)
        want = run(x)
        torch.cuda.synchronize()
        xin.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), f"replay {i} differs from the eager result"
    assert not fused.cluster_exchange_failed()


def test_gemm_ln_cluster_bounded_wait_gives_up_and_recovers():
    """The wait for the partners is bounded: with a limit of one poll some waves of a launch give up
    (the kernel still ends normally, the error word is set, the output is not to be used); with the
    default limit restored and the word cleared the same workspace serves the next call."""
    M, N, K = 8192, 768, 768
    x = _rand(M, K, seed=40); W = _rand(K, N, seed=41, scale=0.05); b = _rand(N, seed=42, scale=0.5)
    r = _rand(M, N, seed=43); gm = (1 + 0.1 * _rand(N, seed=44).float()).half(); bt = _rand(N, seed=45, scale=0.1)
    args = (x.cuda(), fused.pack_weight(W.cuda()), b.cuda(), r.cuda(), gm.cuda(), bt.cuda(), 1e-5)
    want = oe.gemm_bias_residual_layernorm(x, W, b, r, gm, bt, 1e-5)
    _close(fused.gemm_bias_residual_layernorm(*args, form="cluster"), want, "before")
    for _ in range(5):                           # (a single launch in which every wave finds its partners at once is conceivable)
        fused.gemm_bias_residual_layernorm(*args, form="cluster", spin_limit=1)
    torch.cuda.synchronize()                     # the launches end although waves gave up
    assert fused.cluster_exchange_failed()
    with pytest.raises(fused.StofError):         # what the layer / stack / bench call where they synchronise
        fused.check_cluster_exchange()
    assert not fused.cluster_exchange_failed()   # (the check cleared the word)
    _close(fused.gemm_bias_residual_layernorm(*args, form="cluster"), want, "after")
    fused.check_cluster_exchange()
    with pytest.raises(fused.StofError):
        fused.gemm_bias_residual_layernorm(*args, form="cluster", spin_limit=-1)


def test_layer_check_flag_raises_after_a_failed_exchange():
    """EncoderLayer(check=True) surfaces a failed exchange of any earlier cluster launch on the device."""
    from stof import configs, masks as pm
    from stof.layer import EncoderLayer
    B, S, D, H, F = 8, 512, 768, 12, 3072
    w = {k: v.cuda() for k, v in configs.layer_weights(D, F, seed=0).items()}
    x = configs.layer_input(configs.LayerConfig("t", B, S, D, H, F, 1), seed=1, device="cuda")
    lut = pm.get_sparse_storage(configs.mask_c1(S).float()[None].cuda(), 64, 64)[1:]
    layer = EncoderLayer(w, H, eps=1e-12, ln_fusion="cluster")
    layer(x, lut, check=True)                    # a clean run passes
    # the condition is forced from the host: the error word of the workspace the layer's launches use is
    # set as a wave that gave up would set it (the kernel's own give-up path is the test above)
    torch.cuda.synchronize()
    words = [ws for (d, _), ws in fused._cluster_ws.items() if d == x.device.index]
    assert words, "the layer ran no cluster-form launch"
    for ws in words:
        ws[:4].view(torch.int32).fill_(1)
    with pytest.raises(fused.StofError):
        layer(x, lut, check=True)
    layer(x, lut, check=True)                    # the check cleared the word
