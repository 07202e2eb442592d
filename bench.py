#!/usr/bin/env python3
"""Benchmark of the STOF hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

One "step" is one launch of block-masked multi-head attention on workload C4 (fp16,
B2 H16 S4096 D64, causal sliding window of 512 plus every fourth key block, 946 active 64x64
blocks of 4096: the largest single-GPU attention workload and the one the MFMA target is
quoted on), inputs resident in HBM.  The timed region is K steps between device synchronisations; the same
region is bracketed by HIP events on the launch stream for the per-launch kernel time that
the roofline figure uses.  One JSON line is printed:

  value        TFLOP/s counted on ACTIVE blocks only (4*64*64*64 FLOP per block, per batch
               and head: QK^T and PV), whole job, wall clock
  roofline     the attention kernel against the MI355X dense fp16 MFMA peak (2.5 PFLOP/s)
  cpu_baseline the reference's PyTorch-native dense attention (restated in oracle/) timed on
               this machine's host cores on the same workload, in the same unit
  also         the other workloads: C1 (S512, with the host fp32 reference), C2 (B8 H12 S1024), the
               C3 BERT-base encoder layer and the C5 24-layer stack (fused vs PyTorch-ROCm eager,
               ms, per-stage breakdown for C3, output checked against the eager result), the
               HBM-bound kernels and the LUT build
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "sc25-stof-ad_amd"))

import torch  # noqa: E402

PEAK_FP16_TFLOPS = 2500.0     # MI355X dense fp16 matrix peak (published)
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E peak (published)
FLOP_PER_BLOCK = 4 * 64 * 64 * 64

# HBM bytes per launch of the headline kernel come from two counter runs of this script
# (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, each scaled by the same counter on the 256 MiB
# copy of --copy-probe); their summary is a text file under profiles/ whose line
# "traffic_bytes_per_launch: <bytes>" is read here, so the figure reported is the one the
# committed profile holds and names its source.
TRAFFIC_PROFILE = os.path.join("profiles", "block_attn_C4_hbm_traffic.txt")


def measured_traffic():
    """(bytes per launch, source) from the committed counter summary, or (None, reason)."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0]), TRAFFIC_PROFILE
    except OSError:
        pass
    return None, f"{TRAFFIC_PROFILE} not found or without a traffic_bytes_per_launch line"


def attn_setup(cfg, mask_fn, device):
    from stof import configs, masks as pm
    mask = mask_fn(cfg.seq)
    q, k, v = configs.qkv(cfg, seed=0, device=device)
    lut = pm.get_sparse_storage(mask.float()[None].to(device), 64, 64)[1:]
    n_active = int(lut[5][-1])
    return q, k, v, lut, n_active, mask


SETTLE_MS = 80.0   # the GPU's clocks take tens of ms of load to settle (first launches run ~25 % slower)
FLOP_PER_CLK_PER_CU = 4096    # dense fp16 MFMA: 4 SIMDs x 1024 FLOP per clock (32x32x16 in 32 clocks)


class ClockProbe:
    """Shader clock under load, measured in the run: the library's one-wave probe kernel
    (stof_probe_clock: shader cycle counter against the constant 100 MHz counter) launched on a
    second stream while the timed kernels run on the first."""

    def __init__(self):
        from stof import _lib
        self.lib = _lib.lib()
        self.out = torch.zeros(3, dtype=torch.int64, device="cuda")
        self.side = torch.cuda.Stream()
        self.samples = []

    def sample(self, iters=2000):
        self.lib.stof_probe_clock(self.out.data_ptr(), iters, self.side.cuda_stream)
        self.side.synchronize()
        cycles, ticks, _ = self.out.tolist()
        if ticks > 0:
            self.samples.append(cycles / ticks * 0.1)

    def ghz(self):
        s = sorted(self.samples)
        return s[len(s) // 2] if s else None


def time_region(fn, steps, warmup, settle_ms=SETTLE_MS, preheat_ms=0.0):
    """(wall ms per step, event ms per step) for `steps` calls after `warmup` untimed ones.
    After the warm-up calls, further untimed calls keep the GPU busy until `settle_ms` of wall
    time have passed, so that every region - ours, PyTorch's, the copies - is timed at settled
    clocks.  The headline region passes settle_ms=0: it runs exactly `warmup` untimed steps right
    before the timed ones, and keeps the GPU under the same load for `preheat_ms` BEFORE those
    (the clocks of an idle GPU need tens of ms of load, however many warm-up steps are asked for)."""
    t_heat = time.perf_counter()
    while preheat_ms > 0 and (time.perf_counter() - t_heat) * 1e3 < preheat_ms:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t_warm = time.perf_counter()
    while settle_ms > 0 and (time.perf_counter() - t_warm) * 1e3 < settle_ms:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


def bench_attn(cfg, mask_fn, steps, warmup, settle_ms=SETTLE_MS, launch_form=None, dtype=torch.float16, probe=None, preheat_ms=0.0):
    from stof.ops import block_attn
    q, k, v, lut, n_active, _ = attn_setup(cfg, mask_fn, "cuda")
    q, k, v = (t.to(dtype) for t in (q, k, v))
    out = torch.empty_like(q)
    block_attn(q, k, v, lut, out=out, launch_form=launch_form)          # packs the partial-block bit masks and lays out the walk once
    wall_ms, ev_ms = time_region(lambda: block_attn(q, k, v, lut, out=out, launch_form=launch_form), steps, warmup, settle_ms, preheat_ms)
    flop = FLOP_PER_BLOCK * cfg.batch * cfg.heads * n_active
    r = {"wall_ms": wall_ms, "kernel_ms": ev_ms, "flop": flop, "active_blocks": n_active,
         "tflops_wall": flop / wall_ms / 1e9, "tflops_kernel": flop / ev_ms / 1e9}
    if probe is not None:
        # the clock the chip holds under this very load: right after the timed region, with the same
        # launches still queued on the first stream, the probe runs on the second
        for _ in range(8):
            for _ in range(200):
                block_attn(q, k, v, lut, out=out, launch_form=launch_form)
            probe.sample()
        torch.cuda.synchronize()
    return r


def probe_issue_mix(steps=4000):
    """The arithmetic of the attention loop alone (library probe stof_probe_issue_mix): ns per
    wave-step and SIMD for the MFMAs only, the vector arithmetic only and both, at 1 .. 4 wavefronts
    per SIMD, with the shader clock read inside each launch; and what that ceiling is in TFLOP/s."""
    from stof import _lib
    lib = _lib.lib()
    cus = lib.stof_device_compute_units()
    out = torch.zeros(3, dtype=torch.int64, device="cuda")
    sink = torch.zeros(256, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for waves in (1, 2, 3, 4):
        row = {"waves_per_simd": waves}
        for parts, name in ((1, "mfma_only"), (2, "valu_only"), (3, "both")):
            fn = lambda: lib.stof_probe_issue_mix(parts, waves, steps, out.data_ptr(), sink.data_ptr(), stream)
            _, ev_ms = time_region(fn, 20, 5, settle_ms=60.0)
            cyc, ticks, _ = out.tolist()
            ns = ev_ms * 1e6 / (steps * waves)
            row[name] = {"ns_per_wave_step": ns, "clock_ghz": cyc / ticks * 0.1 if ticks else None,
                         "cycles_per_wave_step": ns * (cyc / ticks * 0.1) if ticks else None}
        b = row["both"]["ns_per_wave_step"]
        # a wave-step is 32 queries x 64 keys x 64 channels x 4 FLOP; 4 SIMDs per compute unit
        row["ceiling_tflops"] = 4 * cus * (32 * 64 * 64 * 4) / b / 1e3
        row["overlap"] = (row["mfma_only"]["ns_per_wave_step"] + row["valu_only"]["ns_per_wave_step"] - b) / min(
            row["mfma_only"]["ns_per_wave_step"], row["valu_only"]["ns_per_wave_step"])
        rows.append(row)
    return {"cu_count": cus, "steps": steps,
            "mix_per_wave_step": "16 v_mfma_f32_32x32x16_f16, 32 v_fma_f32, 32 v_exp_f32, 16 v_cvt_pk_f16_f32, 16 v_pk_add_f16, "
                                 "16 v_max3_f32 + lazy-max test; no memory, LDS or barrier", "rows": rows}


def host_cost_us(n=2000):
    """Host time of one block_attn call (Python operator + binding + hipLaunchKernel): a loop of
    launches of the small C1 problem with the clock stopped BEFORE the device is waited for."""
    from stof import _lib, configs
    from stof.ops import block_attn
    q, k, v, lut, _, _ = attn_setup(configs.AttnConfig("C1", 1, 12, 512), configs.mask_c1, "cuda")
    out = torch.empty_like(q)
    for _ in range(200):
        block_attn(q, k, v, lut, out=out)
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(n):
            block_attn(q, k, v, lut, out=out)
        dt = (time.perf_counter() - t0) / n * 1e6
        torch.cuda.synchronize()
        best = dt if best is None else min(best, dt)
    # the same launch through stof.ops.BoundAttention (fixed buffers: validation, strides and the LUT look-up done once)
    from stof.ops import BoundAttention
    run = BoundAttention(q, k, v, lut, out=out)
    for _ in range(200):
        run()
    torch.cuda.synchronize()
    bound = None
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(n):
            run()
        dt = (time.perf_counter() - t0) / n * 1e6
        torch.cuda.synchronize()
        bound = dt if bound is None else min(bound, dt)
    return {"block_attn_host_us_per_call": best, "bound_attention_host_us_per_call": bound, "binding": _lib.binding_name()}


def cpu_baseline_attn(cfg, mask_fn, n_active, budget_s=12.0, max_iters=20, min_iters=3):
    """The reference's dense PyTorch attention (oracle.attention.torch_attn_std) in fp32 on the
    host cores; bounded sample of whole-workload iterations."""
    from oracle import attention as oa
    from stof import configs
    cores = os.cpu_count() or 1
    if os.environ.get("OMP_NUM_THREADS"):
        cores = min(cores, int(os.environ["OMP_NUM_THREADS"]))
    torch.set_num_threads(cores)
    q, k, v = configs.qkv(cfg, seed=0, dtype=torch.float32, device="cpu")
    mask = mask_fn(cfg.seq).float()[None]
    oa.torch_attn_std(q, k, v, mask)           # warm-up
    iters, t0 = 0, time.perf_counter()
    while iters < min_iters or (iters < max_iters and (time.perf_counter() - t0) < budget_s):
        oa.torch_attn_std(q, k, v, mask)
        iters += 1
    dt = (time.perf_counter() - t0) / iters
    flop = FLOP_PER_BLOCK * cfg.batch * cfg.heads * n_active
    return {"value": flop / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "ms_per_step": dt * 1e3,
            "sample": f"1 warm-up + {iters} timed full passes of the {cfg.name} workload (dense fp32 "
                      f"softmax(QK^T/8 - 10000(1-M))V, B{cfg.batch} H{cfg.heads} S{cfg.seq} D64, scores materialised), "
                      f"active-block FLOPs / time"}


def output_check(got, want_eager, valid=None, bound=5e-2):
    """The timed path's output against PyTorch-ROCm's eager fp16 result on the same inputs: a
    guard against timing a path that computes something else, not the parity test (the
    eager layer rounds to fp16 at more points than the fused one; parity against the oracle
    is asserted in tests/).  Rows a padding mask leaves without keys are excluded."""
    d = (got.float() - want_eager.float()).abs()
    if valid is not None:
        d = d[valid]
    m = float(d.max())
    ok = bool(torch.isfinite(got.float()).all()) and m <= bound
    if not ok:
        raise RuntimeError(f"bench output check failed: max |fused - eager| = {m:.3e} (bound {bound})")
    return {"max_abs_diff_vs_eager": m, "bound": bound, "ok": ok}


def bench_layer_c3(steps, warmup):
    """BERT-base encoder layer, B16 S512: fused HIP layer vs PyTorch-ROCm eager."""
    from stof import configs, masks as pm
    from stof.layer import EncoderLayer, eager_layer
    cfg = configs.C3
    w = {k: v.cuda() for k, v in configs.layer_weights(cfg.hidden, cfg.ffn, seed=0).items()}
    x = configs.layer_input(cfg, seed=1, device="cuda")
    mask, L = configs.mask_c3(cfg.batch, cfg.seq, 256, seed=0)
    maskg = mask.cuda().half()
    lut = pm.get_sparse_storage_batched(mask.float().cuda(), 64, 64)[1:]
    out = {}
    for fusion in ("auto", "fused", "cluster", "split"):
        layer = EncoderLayer(w, cfg.heads, eps=cfg.eps, ln_fusion=fusion)
        y = layer(x, lut)
        out[fusion + "_ms"], _ = time_region(lambda: layer(x, lut), steps, warmup)
        if fusion == "auto":
            out["auto_runs"] = layer._ln_form(cfg.batch * cfg.seq, cfg.hidden)
            y_auto = y
    with torch.no_grad():
        y_eager = eager_layer(x, w, maskg, cfg.heads, cfg.eps)
        out["eager_ms"], _ = time_region(lambda: eager_layer(x, w, maskg, cfg.heads, cfg.eps), max(steps // 4, 5), 5)
    out["output_check"] = output_check(y_auto, y_eager, valid=(torch.arange(cfg.seq)[None, :] < L[:, None]).cuda())
    # the same layer on bfloat16 tensors (an addition: the reference is fp16 only)
    layer_bf = EncoderLayer({k: v.to(torch.bfloat16) for k, v in w.items()}, cfg.heads, eps=cfg.eps)
    x_bf = x.to(torch.bfloat16)
    out["bf16_ms"], _ = time_region(lambda: layer_bf(x_bf, lut), steps, warmup)
    layer = EncoderLayer(w, cfg.heads, eps=cfg.eps, ln_fusion="auto")
    out["stages_ms"] = {name: time_region(fn, steps, warmup)[1] for name, fn in layer.stages(x, lut)}
    out["layer_ms_without_qkv_gemm"] = sum(v for k, v in out["stages_ms"].items() if k != "qkv_gemm")
    from stof import fused
    fused.check_cluster_exchange()             # a cluster-form LayerNorm GEMM that gave up a wait above would have timed garbage
    best = out["auto_ms"]                      # what ln_fusion="auto", the default, runs
    out["layer_ms"] = best
    out["speedup_vs_eager"] = out["eager_ms"] / best
    flop = 2 * cfg.batch * cfg.seq * cfg.hidden * (3 * cfg.hidden + cfg.hidden + 2 * cfg.ffn)
    out["gemm_tflops_at_layer_ms"] = flop / best / 1e9
    return out


def bench_small_batch_layer(steps, warmup):
    """BERT-base layer at B1 S512 (the C1 mask): five short kernels, so issuing the launches
    costs as much as running them; eager launches vs one HIP-graph replay vs PyTorch eager."""
    from stof import configs, masks as pm
    from stof.layer import CapturedForward, EncoderLayer, eager_layer
    cfg = configs.LayerConfig("C1-layer", 1, 512, 768, 12, 3072, 1)
    w = {k: v.cuda() for k, v in configs.layer_weights(cfg.hidden, cfg.ffn, seed=0).items()}
    x = configs.layer_input(cfg, seed=1, device="cuda")
    mask = configs.mask_c1(cfg.seq)[None]
    lut = pm.get_sparse_storage(mask.float().cuda(), 64, 64)[1:]
    layer = EncoderLayer(w, cfg.heads, eps=cfg.eps)
    run = CapturedForward(layer, x, lut)
    out = {}
    out["launched_ms"], _ = time_region(lambda: layer(x, lut), steps, warmup)
    out["graph_replay_ms"], _ = time_region(lambda: run.graph.replay(), steps, warmup)
    maskg = mask.cuda().half()
    with torch.no_grad():
        out["eager_ms"], _ = time_region(lambda: eager_layer(x, w, maskg, cfg.heads, cfg.eps), steps, warmup)
    out["speedup_vs_eager"] = out["eager_ms"] / min(out["launched_ms"], out["graph_replay_ms"])
    return out


def bench_c1(steps, warmup, with_cpu):
    """C1 (B1 H12 S512, causal window 128 + first 64 tokens global): the GPU kernel on the fp16
    inputs and the reference's dense attention in fp32 on the host, as the config specifies."""
    from stof import configs
    cfg = configs.AttnConfig("C1", 1, 12, 512)
    r = bench_attn(cfg, configs.mask_c1, steps, warmup)
    out = {"gpu_kernel_ms": r["kernel_ms"], "gpu_tflops": r["tflops_kernel"], "active_blocks": r["active_blocks"]}
    # A launch this short is paced by the host's call (about 11 us from Python): 25 launches
    # recorded into one HIP graph give the time of the kernel itself.
    from stof.ops import block_attn
    q, k, v, lut, _, _ = attn_setup(cfg, configs.mask_c1, "cuda")
    o = torch.empty_like(q)
    block_attn(q, k, v, lut, out=o)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(25):
            block_attn(q, k, v, lut, out=o)
    _, ev = time_region(graph.replay, max(steps // 25, 4), 4)
    out["gpu_kernel_ms_in_graph"] = ev / 25
    out["gpu_tflops_in_graph"] = r["flop"] / (ev / 25) / 1e9
    if with_cpu:
        c = cpu_baseline_attn(cfg, configs.mask_c1, r["active_blocks"], budget_s=3.0, max_iters=50)
        out["cpu_fp32_ms"] = c["ms_per_step"]; out["cpu_tflops"] = c["value"]; out["cpu_cores"] = c["cores"]
    return out


def bench_stack_c5(steps, warmup):
    """C5: 24 post-LN encoder layers, hidden 1024, 16 heads, FFN 4096, B4 S2048, causal window
    256 + first 64 tokens global; whole stack, fused vs PyTorch-ROCm eager."""
    from stof import configs, masks as pm
    from stof.layer import EncoderStack, eager_layer
    cfg = configs.C5
    ws = [{k: v.cuda() for k, v in configs.layer_weights(cfg.hidden, cfg.ffn, seed=i).items()} for i in range(cfg.layers)]
    x = configs.layer_input(cfg, seed=1, device="cuda")
    mask = configs.mask_c5(cfg.seq)
    lut = pm.get_sparse_storage(mask.float()[None].cuda(), 64, 64)[1:]
    stack = EncoderStack(ws, cfg.heads, eps=cfg.eps)
    y = stack(x, lut)
    ms, _ = time_region(lambda: stack(x, lut), steps, warmup)
    maskg = mask.half()[None].cuda()

    def eager():
        h = x
        for w in ws:
            h = eager_layer(h, w, maskg, cfg.heads, cfg.eps)
        return h
    from stof import fused
    fused.check_cluster_exchange()
    with torch.no_grad():
        check = output_check(y, eager(), bound=1e-1)     # 24 chained fp16 layers on both sides
        eager_ms, _ = time_region(eager, max(steps // 2, 3), 2)
    gemm_flop = 2 * cfg.batch * cfg.seq * cfg.hidden * (3 * cfg.hidden + cfg.hidden + 2 * cfg.ffn) * cfg.layers
    return {"stack_ms": ms, "ms_per_layer": ms / cfg.layers, "eager_ms": eager_ms, "speedup_vs_eager": eager_ms / ms,
            "gemm_tflops_at_stack_ms": gemm_flop / ms / 1e9, "layers": cfg.layers,
            "auto_runs": stack.layers[0]._ln_form(cfg.batch * cfg.seq, cfg.hidden), "output_check": check}


def bench_dense_vs_sdpa(steps, warmup):
    """The same kernel on unmasked and causal attention (row-wise front-end: key blocks from index
    arithmetic, no LUT) next to PyTorch-ROCm's fused scaled_dot_product_attention, B16 H16 S4096:
    what the tile engine reaches without mask irregularity, and what the vendor path reaches."""
    import torch.nn.functional as F
    from stof import configs
    from stof.ops import rowwise_attn_full_op
    cfg = configs.AttnConfig("dense", 16, 16, 4096)
    q, k, v = configs.qkv(cfg, seed=0, device="cuda")
    n = cfg.seq // 64
    out = {}
    for causal in (False, True):
        blocks = n * (n + 1) // 2 if causal else n * n
        flop = FLOP_PER_BLOCK * cfg.batch * cfg.heads * blocks
        _, ms = time_region(lambda: rowwise_attn_full_op(q, k, v, causal), steps, warmup)
        _, ms_ref = time_region(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=causal), steps, warmup)
        out["causal" if causal else "full"] = {"kernel_ms": ms, "tflops": flop / ms / 1e9, "frac_mfma_peak": flop / ms / 1e9 / PEAK_FP16_TFLOPS,
                                               "torch_sdpa_ms": ms_ref, "torch_sdpa_tflops": flop / ms_ref / 1e9}
    return out


def bench_hbm_kernels(steps, warmup):
    """HBM-bound kernels: bias+residual+LayerNorm (3 x M x N x 2 bytes) at the C3 size and at a
    size large enough to leave the launch-latency regime, and the fp16 mask -> bit-row pack."""
    from stof import fused
    from stof.ops import pack_mask_bits
    out = {}
    g = torch.Generator().manual_seed(0)
    for tag, M, N in (("bias_res_ln", 8192, 768), ("bias_res_ln_M131072", 131072, 768)):
        x = torch.randn(M, N, generator=g).half().cuda(); r = torch.randn(M, N, generator=g).half().cuda()
        b = torch.randn(N, generator=g).half().cuda()
        _, ev = time_region(lambda: fused.bias_residual_layernorm(x, b, r, b, b, 1e-12), steps, warmup)
        nbytes = 3 * M * N * 2
        out[tag] = {"ms": ev, "GBs": nbytes / ev / 1e6, "frac_hbm": nbytes / ev / 1e6 / PEAK_HBM_GBS, "shape": [M, N],
                    "copy_same_bytes": same_size_copy(nbytes)}
        del x, r
    # what a plain device copy reaches on this machine (read + write of 256 MiB each way)
    src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    _, evc = time_region(lambda: dst.copy_(src), 20, 5)
    out["device_copy_256MiB"] = {"ms": evc, "GBs": 2 * src.numel() / evc / 1e6,
                                 "frac_hbm": 2 * src.numel() / evc / 1e6 / PEAK_HBM_GBS}
    del src, dst
    S = 4096
    m = (torch.rand(S, S, generator=g) < 0.5).half().cuda()
    _, ev2 = time_region(lambda: pack_mask_bits(m, additive=False), steps, warmup)
    pk_bytes = S * S * 2 + S * S // 8
    out["pack_mask_bits"] = {"ms": ev2, "GBs": pk_bytes / ev2 / 1e6, "frac_hbm": pk_bytes / ev2 / 1e6 / PEAK_HBM_GBS,
                             "shape": [S, S], "copy_same_bytes": same_size_copy(pk_bytes)}
    return out


def same_size_copy(nbytes):
    """A plain device copy moving the same number of bytes (half read, half written) as an
    HBM-bound kernel: what the machine gives at that size, launch ramp included."""
    half = max(int(nbytes) // 2, 16)
    src = torch.empty(half, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    _, ev = time_region(lambda: dst.copy_(src), 200, 20)
    return {"ms": ev, "GBs": 2 * half / ev / 1e6, "frac_hbm": 2 * half / ev / 1e6 / PEAK_HBM_GBS, "bytes": 2 * half}


def bench_lut_build(with_cpu, steps=200):
    """Block LUT of the C4 mask (S 4096, 64 x 64 blocks) built by the GPU kernels: the whole
    get_sparse_storage call (exactly shaped tensors: one device -> host read of the list lengths,
    plus the reference's nnz figure and additive fp16 blocks), and the two kernels alone
    (build_lut_device: no synchronisation; HBM-bound, S^2 x element bytes read once); next to
    the reference's Python double loop (restated in oracle/) on the host at S 2048."""
    from stof import configs, masks as pm
    out = {}
    for tag, dtype in (("fp16", torch.float16), ("fp32", torch.float32)):
        mask = configs.mask_c4(4096).to(dtype)[None].cuda()
        pm.get_sparse_storage(mask, 64, 64)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            pm.get_sparse_storage(mask, 64, 64)
        torch.cuda.synchronize()
        out[f"get_sparse_storage_ms_S4096_{tag}"] = (time.perf_counter() - t0) / 20 * 1e3
        # the two kernels with every buffer allocated beforehand (what a serving loop would do)
        from stof import _lib
        lib = _lib.lib()
        S, tiles = 4096, 64 * 64
        i32 = lambda n: torch.empty(n, dtype=torch.int32, device="cuda")
        frp, prp, lrp, fci, pci, lci, counts = i32(65), i32(65), i32(65), i32(tiles), i32(tiles), i32(tiles), i32(4)
        bits = torch.empty(tiles * 64, dtype=torch.int64, device="cuda")
        ws = torch.empty(lib.stof_build_lut_workspace_bytes(S, 64, 64), dtype=torch.uint8, device="cuda")
        m2d = mask[0]
        stream = torch.cuda.current_stream().cuda_stream
        args = (m2d.data_ptr(), m2d.element_size(), S, S, 64, 64, frp.data_ptr(), fci.data_ptr(), prp.data_ptr(), pci.data_ptr(),
                lrp.data_ptr(), lci.data_ptr(), bits.data_ptr(), counts.data_ptr(), tiles, tiles, tiles, ws.data_ptr(), ws.numel(), stream)
        _, ev = time_region(lambda: lib.stof_build_lut(*args), steps, 20)
        assert counts.tolist() == [840, 106, 946, 0]
        nbytes = 4096 * 4096 * mask.element_size()
        out[f"kernels_ms_S4096_{tag}"] = ev
        out[f"kernels_GBs_{tag}"] = nbytes / ev / 1e6
        out[f"kernels_frac_hbm_{tag}"] = nbytes / ev / 1e6 / PEAK_HBM_GBS
        out[f"copy_same_bytes_{tag}"] = same_size_copy(nbytes)
    out["gpu_ms_S4096"] = out["kernels_ms_S4096_fp16"]
    if with_cpu:
        from oracle import masks as om
        m2 = configs.mask_c4(2048).float()[None].numpy()
        t0 = time.perf_counter()
        om.get_sparse_storage(m2, 64, 64)
        out["cpu_loop_ms_S2048"] = (time.perf_counter() - t0) * 1e3
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=2000,
                    help="untimed steps before the timed ones; the default (about 70 ms of load) lets the clocks settle")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="ms of the same load run BEFORE the warm-up steps of the headline, so that a small --warmup is not "
                         "timed on the clock ramp of an idle GPU (0 = none); reported as config.clock_settle_ms")
    ap.add_argument("--no-extras", action="store_true", help="skip everything but the C4 attention step")
    ap.add_argument("--extras", default="c1,c2,c5attn,c4big,forms,dense,c3,c3small,c5,hbm,lut",
                    help="comma-separated subset of the extra workloads to run (for profiling one kind of kernel)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--probe-mix", action="store_true",
                    help="run only the instruction-mix probe of the attention loop and print its table as JSON")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain device copy of 256 MiB, so that a counter run of this "
                         "command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the hot path shards by batch x head with no "
              "exchange step; nothing here uses a second device). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback.", file=sys.stderr)
        sys.exit(2)

    from stof import configs
    torch.cuda.set_device(0)
    if args.probe_mix:
        print(json.dumps(probe_issue_mix()))
        return
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    from stof import _lib
    probe = ClockProbe()
    cus = _lib.lib().stof_device_compute_units()
    # the GPU is kept under this load for --settle-ms first (clock ramp of an idle device), then exactly W warm-up steps, then K timed
    c4 = bench_attn(configs.C4, configs.mask_c4, args.steps, args.warmup, settle_ms=0, probe=probe, preheat_ms=args.settle_ms)
    clock = probe.ghz()
    traffic, traffic_source = measured_traffic()
    line = {
        "metric": "masked-MHA TFLOP/s (active blocks) + encoder-layer ms, fp16, 1xMI355X",
        "value": c4["tflops_wall"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": c4["wall_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "C4: long-sequence block-masked MHA, B2 H16 S4096 D64, causal sliding window of 512 + "
                               "every 4th key block, 64 x 64 blocks", "active_blocks": c4["active_blocks"],
                   "blocks_total": (configs.C4.seq // 64) ** 2, "block": 64, "flop_per_step": c4["flop"],
                   "clock_settle_ms": args.settle_ms},
        "roofline": {"bound": "mfma", "achieved": c4["tflops_kernel"], "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": c4["tflops_kernel"] / PEAK_FP16_TFLOPS, "traffic": traffic, "traffic_source": traffic_source,
                     "algorithmic_bytes": 4 * configs.C4.batch * configs.C4.heads * configs.C4.seq * 64 * 2,
                     "kernel": "block_attn_fwd_kernel", "kernel_ms": c4["kernel_ms"],
                     # what was measured on this box in this run, next to the published peak the fraction divides by:
                     # compute units (hipDeviceGetAttribute) and the shader clock under the timed load (the library's
                     # probe kernel on a second stream: shader cycle counter against the 100 MHz counter, median of 8)
                     "cu_count": cus, "clock_ghz_under_load": clock,
                     "peak_at_measured_clock": (cus * FLOP_PER_CLK_PER_CU * clock / 1e3) if clock else None,
                     "frac_at_measured_clock": (c4["tflops_kernel"] / (cus * FLOP_PER_CLK_PER_CU * clock / 1e3)) if clock else None},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_attn(configs.C4, configs.mask_c4, c4["active_blocks"])
    if not args.no_extras:
        also = {}
        want = set(args.extras.split(","))
        also["host"] = host_cost_us()
        if "c2" in want:
            c2 = bench_attn(configs.C2, configs.mask_c2, args.steps, args.warmup)
            also["C2_mha_S1024"] = {"tflops": c2["tflops_kernel"], "frac_mfma_peak": c2["tflops_kernel"] / PEAK_FP16_TFLOPS,
                                    "kernel_ms": c2["kernel_ms"], "active_blocks": c2["active_blocks"]}
        if "c5attn" in want:
            c5a = bench_attn(configs.AttnConfig("C5-attention", 4, 16, 2048), configs.mask_c5, args.steps, args.warmup)
            also["C5_attention_B4_H16_S2048"] = {"tflops": c5a["tflops_kernel"], "frac_mfma_peak": c5a["tflops_kernel"] / PEAK_FP16_TFLOPS,
                                                 "kernel_ms": c5a["kernel_ms"], "active_blocks": c5a["active_blocks"]}
        if "c4big" in want:
            big = configs.AttnConfig("C4x8", 16, 16, 4096)
            c4b = bench_attn(big, configs.mask_c4, max(args.steps // 4, 10), 5)
            also["C4_mask_B16_H16"] = {"tflops": c4b["tflops_kernel"], "frac_mfma_peak": c4b["tflops_kernel"] / PEAK_FP16_TFLOPS,
                                       "kernel_ms": c4b["kernel_ms"]}
        if "forms" in want:
            # the three launch forms on the headline workload (the default picks by grid size)
            also["C4_launch_forms_kernel_ms"] = {
                form: bench_attn(configs.C4, configs.mask_c4, max(args.steps // 4, 50), 50, launch_form=form)["kernel_ms"]
                for form in ("two_rows", "key_split", "pipelined")}
            # the same workload on bfloat16 tensors (not the headline: the reference computes in fp16)
            also["C4_bf16_kernel_ms"] = bench_attn(configs.C4, configs.mask_c4, max(args.steps // 4, 50), 50,
                                                   dtype=torch.bfloat16)["kernel_ms"]
        if "dense" in want:
            also["dense_S4096_B16_H16_vs_torch_sdpa"] = bench_dense_vs_sdpa(max(args.steps // 10, 10), 3)
        if "c1" in want:
            also["C1_mha_S512"] = bench_c1(args.steps, args.warmup, not args.no_cpu)
        if "c3" in want:
            also["C3_bert_base_layer"] = bench_layer_c3(max(args.steps // 4, 20), 10)
        if "c3small" in want:
            also["bert_base_layer_B1_S512"] = bench_small_batch_layer(max(args.steps // 4, 20), 20)
        if "c5" in want:
            also["C5_stack_24_layers"] = bench_stack_c5(max(args.steps // 20, 5), 2)
        if "hbm" in want:
            also["hbm_bound"] = bench_hbm_kernels(args.steps, args.warmup)
        if "lut" in want:
            also["lut_build"] = bench_lut_build(not args.no_cpu)
        line["also"] = also
    print(json.dumps(line))


if __name__ == "__main__":
    main()
