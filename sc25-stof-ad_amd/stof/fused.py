"""Fused encoder operators on the HIP library.

Reference-named entry points (same signatures as ``src/triton_template``):

* ``triton_matmul_bias_layernorm(A, B, bias, eps=1e-5)``      gemm_add_layernorm.py:126-144
* ``triton_matmul_batch(a, b, d, bias)``                      gemm_gemm.py:158-174
* ``triton_batched_bias_layernorm(x, bias, weight, bias_ln, eps=1e-5)``  add_layernorm.py:86-107

and the explicit forms the encoder layer uses:

* ``gemm_bias_act(x, Wt, bias, act)``                          act(x @ Wt^T + bias)
* ``gemm_bias_gelu(x, Wt, bias, approximate)``                 the same with torch's name for the GELU variant
* ``gemm_act_gemm(x, W1t, b1, W2t, b2, act)``                  act(x @ W1t^T + b1) @ W2t^T + b2, one launch
* ``gemm_bias_residual_layernorm(x, Wt, bias, residual, gamma, beta, eps)``
* ``bias_residual_layernorm(x, bias, residual, gamma, beta, eps)``

Weights are consumed in the ``[N, K]`` (nn.Linear) orientation, K contiguous, which is what
the MFMA B operand wants; ``pack_weight`` converts a reference-style ``[K, N]`` matrix once.
Nothing here falls back to PyTorch math: a missing library or unsupported shape raises.
"""
import functools

import torch

from . import _lib
from ._lib import StofError, check

ACT = {"none": 0, "gelu": 1, "gelu_erf": 1, "gelu_tanh": 2, "relu": 3}
_PACK_ATTR = "_stof_packed_nk"


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t):
    """Raw handle of torch's current stream on the device of tensor ``t``."""
    if _raw_stream is not None and t.device.index is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _require(cond, msg):
    if not cond:
        raise StofError(msg)


_DTYPES = {torch.float16: 0, torch.bfloat16: 1}   # STOF_DTYPE_*


def _f16c(name, t, allow_none=False, like=None):
    """``t`` contiguous; a CUDA float16 tensor, or of ``like``'s 16-bit format if that is given."""
    if t is None:
        if not allow_none:
            raise StofError(f"{name} is required")
        return None
    want = torch.float16 if like is None else like.dtype
    if not (t.is_cuda and t.dtype == want):
        raise StofError(f"{name} must be a CUDA {str(want).replace('torch.', '')} tensor")
    return t if t.is_contiguous() else t.contiguous()


def _elem16(name, t):
    """``t`` must be a CUDA tensor in one of the two 16-bit formats; its STOF_DTYPE_* code."""
    dt = _DTYPES.get(t.dtype) if t.is_cuda else None
    if dt is None:
        raise StofError(f"{name} must be a CUDA float16 or bfloat16 tensor")
    return dt


def _p(t):
    return None if t is None else t.data_ptr()


def pack_weight(W):
    """Reference-style ``[K, N]`` weight -> ``[N, K]`` contiguous, converted once per tensor
    object and content version (the copy is kept on the tensor)."""
    cached = getattr(W, _PACK_ATTR, None)
    if cached is not None and cached[0] == W._version:
        return cached[1]
    Wt = W.t().contiguous()
    try:
        setattr(W, _PACK_ATTR, (W._version, Wt))
    except AttributeError:
        pass
    return Wt


def bias_residual_layernorm(x, bias, residual, gamma, beta, eps=1e-5, return_stats=False, out=None):
    """LN(x + bias + residual) * gamma + beta over the last dim; any operand but x may be None.
    float16 or, all operands alike, bfloat16."""
    dt = _elem16("x", x)
    if not x.is_contiguous():
        x = x.contiguous()
    N = x.shape[-1]
    M = x.numel() // N
    bias = _f16c("bias", bias, True, x); residual = _f16c("residual", residual, True, x)
    gamma = _f16c("gamma", gamma, True, x); beta = _f16c("beta", beta, True, x)
    for name, t in (("bias", bias), ("gamma", gamma), ("beta", beta)):
        if t is not None and t.numel() != N:
            raise StofError(f"{name} must have {N} elements")
    if residual is not None and residual.shape != x.shape:
        raise StofError("residual must have x's shape")
    if out is not None and not (out.shape == x.shape and out.dtype == x.dtype and out.is_contiguous()):
        raise StofError("out must be contiguous, with x's shape")
    y = torch.empty_like(x) if out is None else out
    mean = rstd = None
    if return_stats:
        mean = torch.empty(M, dtype=torch.float32, device=x.device)
        rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    check(_lib.lib().stof_bias_res_ln_dt(x.data_ptr(), _p(bias), _p(residual), _p(gamma), _p(beta),
                                         y.data_ptr(), _p(mean), _p(rstd), M, N, float(eps), dt, _stream(y)),
          "stof_bias_res_ln")
    return (y, mean, rstd) if return_stats else y


def triton_batched_bias_layernorm(x, bias, weight, bias_ln, eps=1e-5):
    """src/triton_template/add_layernorm.py:86-107: LN(x + bias) * weight + bias_ln, x [B,S,hidden]."""
    return bias_residual_layernorm(x, bias, None, weight, bias_ln, eps)


_splitk_ws = {}           # (device index, stream handle) -> zeroed workspace tensor, grown on demand


def _splitk_workspace(dev, stream, nbytes):
    """A workspace for stof_gemm_bias_act_splitk, one per (device, stream), zero at first use:
    every call leaves its counters zero again, and calls on one stream do not overlap."""
    key = (dev.index, stream)
    ws = _splitk_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 23), dtype=torch.uint8, device=dev)
        _splitk_ws[key] = ws
    return ws


def gemm_bias_act(x, Wt, bias=None, act="none", out=None, splits=None):
    """act(x @ Wt^T + bias): x [..., K] (rows may be strided), Wt [N, K], bias [N]; float16 or,
    all operands alike, bfloat16.

    ``splits``: None = the library's rule (stof_gemm_bias_act_splitk_plan: K split over several
    workgroups per tile where the output has few tiles and K is long), 1 = one workgroup per tile
    (stof_gemm_bias_act), 2 .. 8 = that many splits (stof_gemm_bias_act_splitk)."""
    if act not in ACT:
        raise StofError(f"unknown activation {act!r}")
    if splits is not None and not 1 <= int(splits) <= 8:
        raise StofError("splits must be None or 1 .. 8")
    dt = _elem16("x", x)
    Wt = _f16c("Wt", Wt, like=x); bias = _f16c("bias", bias, True, x)
    K = x.shape[-1]
    N = Wt.shape[0]
    if Wt.dim() != 2 or Wt.shape[1] != K:
        raise StofError(f"Wt must be [N, {K}]")
    if bias is not None and bias.numel() != N:
        raise StofError(f"bias must have {N} elements")
    # rows of x: dense tensors (the usual case) are addressed as they are, others through a 2-D view
    if x.is_contiguous():
        x2, lda = x, K
    else:
        x2 = x if x.dim() == 2 else x.reshape(-1, K)
        if x2.stride(1) != 1:
            x2 = x2.contiguous()
        lda = x2.stride(0)
    M = x.numel() // K
    if out is None:
        out = torch.empty(x.shape[:-1] + (N,), dtype=x.dtype, device=x.device)
        o2, ldc = out, N
    else:
        if out.dtype != x.dtype:
            raise StofError("out must have x's element format")
        o2 = out if out.dim() == 2 else out.view(-1, N)
        if o2.shape[0] != M or o2.stride(1) != 1:
            raise StofError("out must be [..., N] with contiguous rows")
        ldc = o2.stride(0)
    lib = _lib.lib()
    st = _stream(o2)
    if splits is None:
        splits = _splitk_plan(M, N, K)
    if splits > 1:
        nbytes = lib.stof_gemm_bias_act_splitk_workspace_bytes(M, N, splits)
        _require(nbytes > 0, f"shape not supported by the split-K form: M {M}, N {N}")
        ws = _splitk_workspace(x.device, st, nbytes)
        check(lib.stof_gemm_bias_act_splitk_dt(x2.data_ptr(), Wt.data_ptr(), _p(bias), o2.data_ptr(),
                                               M, N, K, lda, ldc, ACT[act], int(splits),
                                               ws.data_ptr(), ws.numel(), dt, st),
              "stof_gemm_bias_act_splitk")
        return out
    check(lib.stof_gemm_bias_act_dt(x2.data_ptr(), Wt.data_ptr(), _p(bias), o2.data_ptr(),
                                    M, N, K, lda, ldc, ACT[act], dt, st),
          "stof_gemm_bias_act")
    return out


def gemm_bias_gelu(x, Wt, bias=None, approximate="none", out=None):
    """GELU(x @ Wt^T + bias) with torch's naming of the variant: ``approximate`` "none" (erf, BERT,
    src/benchmk_end2end.py:81) or "tanh" (GPT, :25-26)."""
    _require(approximate in ("none", "tanh"), f"approximate must be 'none' or 'tanh', got {approximate!r}")
    return gemm_bias_act(x, Wt, bias, "gelu" if approximate == "none" else "gelu_tanh", out=out)


_cluster_ws = {}          # (device index, stream handle) -> zeroed workspace tensor, grown on demand


def cluster_supported(N, K):
    """Shapes the row-block-cluster form of the LayerNorm GEMM takes."""
    return N % 128 == 0 and 256 <= N <= 1024 and K % 64 == 0


def _cluster_workspace(dev, stream, nbytes):
    """Workspace of stof_gemm_bias_res_ln_cluster, one per (device, stream): its counters start
    as zeros and every call leaves them zero again; calls on one stream do not overlap."""
    key = (dev.index, stream)
    ws = _cluster_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 21), dtype=torch.uint8, device=dev)
        _cluster_ws[key] = ws
    return ws


def check_cluster_exchange(dev=None):
    """Raise ``StofError`` if a bounded wait inside any cluster-form LayerNorm GEMM launched on
    ``dev`` since the last check ran out (the rows that launch wrote are then invalid), and put
    the error word back to zero.  The word stays set until it is cleared, so ONE check after a
    batch of work covers every launch of that batch.  Synchronises the device: call it where the
    caller synchronises anyway (``EncoderLayer`` / ``EncoderStack`` / ``CapturedForward`` do so
    with ``check=True``).  The waits only run out when something else keeps compute units
    occupied for about a tenth of a second while the kernel runs - another stream's or another
    process's long kernel; on a device of one's own they cannot."""
    if cluster_exchange_failed(dev):
        clear_cluster_exchange_error(dev)
        raise StofError("a LayerNorm GEMM in its cluster form gave up waiting for a partner workgroup (the device was "
                        "shared with a long-running kernel?): the outputs since the last check are invalid. Use "
                        "ln_fusion='split' / form='split' where the device is shared.")


def cluster_exchange_failed(dev=None):
    """True if a wait inside any cluster-form launch on ``dev`` ran out (its output is then
    invalid): the first word of the workspace.  Synchronises the device."""
    dev = torch.device("cuda", torch.cuda.current_device()) if dev is None else torch.device(dev)
    torch.cuda.synchronize(dev)
    return any(bool(ws[:4].view(torch.int32).item()) for (d, _), ws in _cluster_ws.items() if d == dev.index)


def clear_cluster_exchange_error(dev=None):
    """Put the error word of every cluster workspace on ``dev`` back to zero."""
    dev = torch.device("cuda", torch.cuda.current_device()) if dev is None else torch.device(dev)
    for (d, _), ws in _cluster_ws.items():
        if d == dev.index:
            ws[:4].zero_()


# From this many 128 x 128 output tiles on, the LayerNorm GEMM runs its cluster form.  Measured on
# MI355X, us, cluster / GEMM then LayerNorm kernel / row form, rows x N x K: 8192 x 768 x 768
# 22.3 / 26.0 / 42.5, 8192 x 768 x 3072 51.9 / 53.0 / 112, 8192 x 1024 x 4096 74.4 / 79.5 / 197,
# 16384 x 768 x 768 37.9 / 42.2 / 49.0, 65536 x 1024 x 1024 221 / 237 / 288, 65536 x 512 x 512
# 61 / 78 / 84; with K = 4 N the two-launch form is level with it or up to 7 % ahead from 32768
# rows on (32768 x 768 x 3072 207 / 193 / 277, 32768 x 1024 x 4096 320 / 309 / 503, 65536 x 768 x 3072
# 394 / 394 / 558: with several tiles per workgroup each tile's wait for its partners costs more
# than the LayerNorm kernel's second pass).  Below, the tiled GEMM
# runs its 64-token form, which the cluster kernel has no counterpart of: 2048 x 768 x 3072
# (96 tiles) 38 / 28 / 108.  The row form (one workgroup per 64 rows streams the whole weight
# matrix) is level with the others only at N 256.
CLUSTER_MIN_TILES = 192


@functools.lru_cache(maxsize=4096)
def _splitk_plan(M, N, K):
    """stof_gemm_bias_act_splitk_plan, remembered per shape (a pure function of the three sizes)."""
    return _lib.lib().stof_gemm_bias_act_splitk_plan(M, N, K)


@functools.lru_cache(maxsize=4096)
def ln_gemm_form(M, N, K):
    """How ``form="auto"`` runs a LayerNorm GEMM of M rows: "cluster", or "split" (tiled GEMM, then
    the bias+residual+LayerNorm kernel; the pre-normalisation values pass through HBM as fp16), or
    "row" where K is a multiple of 32 but not of 64, which only that kernel takes."""
    tiles = ((M + 127) // 128) * (N // 128)
    # (where the tiled GEMM would split K - 129 .. 192 tiles and a long K - it overtakes the cluster
    # form, which cannot: 4096 x 768 x 3072 36.5 us as two launches against 39.9)
    if cluster_supported(N, K) and tiles >= CLUSTER_MIN_TILES and _splitk_plan(M, N, K) == 1:
        return "cluster"
    return "split" if K % 64 == 0 else "row"


def gemm_bias_residual_layernorm(x, Wt, bias, residual, gamma, beta, eps=1e-5, out=None, form="auto", spin_limit=0):
    """LN(x @ Wt^T + bias + residual) * gamma + beta.

    The cluster form (what ``"auto"`` takes from 192 output tiles of 128 x 128 on) assumes a
    device that is not shared with long-running kernels of other streams or processes: its
    workgroups wait for one another, boundedly; a wait that runs out leaves invalid rows and
    sets an error word that ``check_cluster_exchange`` reads.  ``spin_limit`` (polls, 0 = the
    library's 2^18) is for tests of that path.

    ``form="row"``: one workgroup owns the whole row of N features (stof_gemm_bias_res_ln).
    ``form="cluster"``: the N / 128 workgroups of a block of 128 token rows each own 128 features
    and exchange per-row statistics through a small workspace (stof_gemm_bias_res_ln_cluster).
    In both the pre-normalisation values stay in registers.
    ``form="split"``: stof_gemm_bias_act, then stof_bias_residual_layernorm.
    ``form="auto"``: ``ln_gemm_form`` chooses."""
    if form not in ("auto", "row", "cluster", "split"):
        raise StofError(f"unknown form {form!r}")
    if form == "auto":
        form = ln_gemm_form(x.numel() // x.shape[-1], Wt.shape[0], x.shape[-1])
    if form == "split":
        y = gemm_bias_act(x, Wt, None, "none")
        if residual is not None and residual.shape != y.shape:
            residual = residual.reshape(y.shape)
        return bias_residual_layernorm(y, bias, residual, gamma, beta, eps, out=out)
    dt = _elem16("x", x)
    if dt != 0 and form != "cluster":
        raise StofError("the row form takes float16 only")
    if not x.is_contiguous():
        x = x.contiguous()
    Wt = _f16c("Wt", Wt, like=x)
    bias = _f16c("bias", bias, True, x); residual = _f16c("residual", residual, True, x)
    gamma = _f16c("gamma", gamma, True, x); beta = _f16c("beta", beta, True, x)
    K = x.shape[-1]
    N = Wt.shape[0]
    M = x.numel() // K
    if Wt.dim() != 2 or Wt.shape[1] != K:
        raise StofError(f"Wt must be [N, {K}]")
    if residual is not None and residual.numel() != M * N:
        raise StofError("residual must be [..., N] matching x's rows")
    for name, t in (("bias", bias), ("gamma", gamma), ("beta", beta)):
        if t is not None and t.numel() != N:
            raise StofError(f"{name} must have {N} elements")
    if out is None:
        out = torch.empty(x.shape[:-1] + (N,), dtype=x.dtype, device=x.device)
    elif not (out.dtype == x.dtype and out.device == x.device and tuple(out.shape) == tuple(x.shape[:-1]) + (N,) and out.is_contiguous()):
        raise StofError(f"out must be a contiguous {tuple(x.shape[:-1]) + (N,)} tensor of x's element format on x's device")
    lib = _lib.lib()
    st = _stream(out)
    if form == "cluster":
        _require(cluster_supported(N, K), f"unsupported shape for the cluster form: N {N}, K {K}")
        nbytes = lib.stof_gemm_bias_res_ln_cluster_workspace_bytes(M, N)
        ws = _cluster_workspace(x.device, st, nbytes)
        check(lib.stof_gemm_bias_res_ln_cluster_bounded(x.data_ptr(), Wt.data_ptr(), _p(bias), _p(residual), _p(gamma), _p(beta),
                                                        out.data_ptr(), M, N, K, K, N, N, float(eps),
                                                        ws.data_ptr(), ws.numel(), dt, int(spin_limit), st),
              "stof_gemm_bias_res_ln_cluster")
        return out
    check(lib.stof_gemm_bias_res_ln(x.data_ptr(), Wt.data_ptr(), _p(bias), _p(residual),
                                    _p(gamma), _p(beta), out.data_ptr(), M, N, K, float(eps), st),
          "stof_gemm_bias_res_ln")
    return out


def triton_matmul_bias_layernorm(A, B, bias, eps=1e-5):
    """src/triton_template/gemm_add_layernorm.py:126-144: LayerNorm WITHOUT gamma/beta of
    ``A[b,M,K] @ B[b,K,N] + bias``.

    ``B`` is the reference's per-batch weight, always an ``expand`` of one ``[K,N]`` matrix at
    its call sites (src/tuning_STOF_cost.py:59-60); a batch of distinct matrices is rejected.
    ``bias`` of N elements is a bias; of shape ``[b,M,N]`` it is the caller's
    ``bias + residual`` (same call sites) and is added element-wise - the evident intent,
    where the reference kernel reads only its first N elements.
    """
    _require(A.dim() == 3 and B.dim() == 3 and A.shape[2] == B.shape[1], "A [b,M,K], B [b,K,N] expected")
    _require(B.stride(0) == 0 or B.shape[0] == 1, "B must be one weight matrix expanded over the batch")
    N = B.shape[2]
    Wt = pack_weight(B[0])
    if bias.numel() == N:
        return gemm_bias_residual_layernorm(A, Wt, bias.reshape(N), None, None, None, eps)
    _require(bias.shape == A.shape[:2] + (N,), "bias must have N elements or shape [b,M,N]")
    return gemm_bias_residual_layernorm(A, Wt, None, bias, None, None, eps)


# Rows up to which "auto" callers take the single-launch chained form.  0: never - measured on
# MI355X it loses to two GEMM launches at every row count tried (M 256 / 512 / 1024 at K 768,
# F 3072: 50 / 67 / 101 us against 30 / 31 / 35 us), see csrc/ffn_chain_gfx950.hip.
CHAIN_MAX_ROWS = 0
_chain_ws = {}            # (device index, stream handle) -> zeroed workspace tensor, grown on demand


def chain_supported(M, K, F, H):
    """Shapes the single-launch chained kernel takes (stof_gemm_act_gemm)."""
    return K % 64 == 0 and F % 128 == 0 and H % 128 == 0


def _chain_workspace(dev, stream, nbytes):
    """A zeroed workspace for stof_gemm_act_gemm, one per (device, stream): every call leaves
    its workspace zero again, and calls on one stream do not overlap."""
    key = (dev.index, stream)
    ws = _chain_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 22), dtype=torch.uint8, device=dev)
        _chain_ws[key] = ws
    return ws


def gemm_act_gemm(x, W1t, b1, W2t, b2=None, act="gelu", out=None):
    """act(x @ W1t^T + b1) @ W2t^T (+ b2) in one launch (stof_gemm_act_gemm): x [..., K],
    W1t [F, K], W2t [H, F]; the [.., F] intermediate is fp16 and stays on chip.  For small row
    counts; K % 64 == 0, F % 128 == 0, H % 128 == 0."""
    _require(act in ACT, f"unknown activation {act!r}")
    _require(x.is_cuda and x.dtype == torch.float16, "x must be a CUDA float16 tensor")
    W1t = _f16c("W1t", W1t); W2t = _f16c("W2t", W2t)
    b1 = _f16c("b1", b1, True); b2 = _f16c("b2", b2, True)
    K = x.shape[-1]
    F, H = W1t.shape[0], W2t.shape[0]
    _require(W1t.dim() == 2 and W1t.shape[1] == K, f"W1t must be [F, {K}]")
    _require(W2t.dim() == 2 and W2t.shape[1] == F, f"W2t must be [H, {F}]")
    _require(b1 is None or b1.numel() == F, f"b1 must have {F} elements")
    _require(b2 is None or b2.numel() == H, f"b2 must have {H} elements")
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    _require(chain_supported(M, K, F, H), f"unsupported shape for the chained kernel: K {K}, F {F}, H {H}")
    if out is None:
        out = torch.empty(x.shape[:-1] + (H,), dtype=torch.float16, device=x.device)
    o2 = out.view(-1, H)
    _require(o2.shape[0] == M and o2.stride(1) == 1, "out must be [..., H] with contiguous rows")
    lib = _lib.lib()
    st = _stream(o2)
    nbytes = lib.stof_gemm_act_gemm_workspace_bytes(M, H)
    ws = _chain_workspace(x.device, st, nbytes)
    check(lib.stof_gemm_act_gemm(x2.data_ptr(), W1t.data_ptr(), _p(b1), W2t.data_ptr(), _p(b2), o2.data_ptr(),
                                 M, K, F, H, x2.stride(0), o2.stride(0), ACT[act], ws.data_ptr(), ws.numel(), st),
          "stof_gemm_act_gemm")
    return out


def triton_matmul_batch(a, b, d, bias, single_launch=None):
    """src/triton_template/gemm_gemm.py:158-174: gelu_tanh(a @ b + bias) @ d, a [B,M,K],
    b [K,N], d [N,H]; the intermediate is fp16 (gemm_gemm.py:152).  ``single_launch=True`` (or a
    row count up to CHAIN_MAX_ROWS) takes the chained kernel that keeps the intermediate on chip;
    the default is two launches of the GEMM kernel with the fp16 intermediate in HBM, which is
    the faster form on MI355X at every size measured."""
    _require(a.dim() == 3 and b.dim() == 2 and d.dim() == 2, "a [B,M,K], b [K,N], d [N,H] expected")
    b1 = bias.reshape(-1)[: b.shape[1]]
    rows = a.shape[0] * a.shape[1]
    fits = chain_supported(rows, a.shape[2], b.shape[1], d.shape[1])
    _require(fits or not single_launch, "shape not supported by the single-launch form (K % 64, F % 128, H % 128)")
    if fits and (single_launch or (single_launch is None and rows <= CHAIN_MAX_ROWS)):
        return gemm_act_gemm(a, pack_weight(b), b1, pack_weight(d), None, "gelu_tanh")
    t = gemm_bias_act(a, pack_weight(b), b1, "gelu_tanh")
    return gemm_bias_act(t, pack_weight(d), None, "none")
