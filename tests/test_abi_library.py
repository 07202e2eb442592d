"""The C-ABI shared library loads and exports every symbol include/stof_abi.h declares, and
its host-side argument checks reject bad calls before any launch (no GPU needed: every call
here fails validation and returns a negative status)."""
import ctypes
import os
import re

import pytest

from stof import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "stof_abi.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(stof_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module", params=["ctypes", "ext"])
def lib(request):
    """Every test of this module runs against both bindings of the C ABI: ctypes on the library
    itself and the pybind11 extension module built beside it."""
    global _BINDING
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libstof_hip.so not built (python sc25-stof-ad_amd/csrc/build.py)")
    h = _lib.lib(request.param)
    if h is None:
        pytest.skip("extension module _stof_ext not built (python sc25-stof-ad_amd/csrc/build.py; needs pybind11)")
    _BINDING = request.param
    return h


_BINDING = "ctypes"


def test_every_declared_symbol_is_exported_and_bound(lib):
    syms = _declared_symbols()
    assert len(syms) >= 8
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for s in syms:
        assert hasattr(raw, s), f"{s} declared in stof_abi.h but not exported"
        assert s in _lib._SIGNATURES, f"{s} has no ctypes signature"
        assert hasattr(lib, s), f"{s} missing from the {_BINDING} binding"
    assert sorted(_lib._SIGNATURES) == syms


def test_the_binding_in_use_is_the_extension_module_when_it_is_built():
    if _lib.lib("ext") is None:
        pytest.skip("extension module not built")
    if os.environ.get("STOF_BINDING", "") == "ctypes":
        pytest.skip("ctypes forced by the environment")
    assert _lib.binding_name() == "ext"


def test_version_and_status_strings(lib):
    assert lib.stof_abi_version() == 4
    for code in (0, -1, -2, -3, -4, -5, -6, -7, -99):
        assert len(lib.stof_status_string(code)) > 0


def _s3(a, b, c):
    return (a, b, c) if _BINDING == "ext" else (ctypes.c_int64 * 3)(a, b, c)


def test_block_attn_argument_checks(lib):
    st = _s3(12 * 128 * 64, 128 * 64, 64)
    P = 4096   # fake, 16-byte aligned, never dereferenced: validation fails first
    call = lambda **kw: lib.stof_block_attn_fwd(
        kw.get("q", P), P, P, P, P, P, P, P, P, P, P, kw.get("bm", 64), kw.get("bn", 64), 0.125,
        kw.get("qs", st), st, st, st, 1, kw.get("S", 128), 12, kw.get("D", 64), kw.get("dtype", 0), kw.get("lbs", 0), kw.get("form", -1), None)
    assert call(q=None) == -1            # NULL pointer
    assert call(S=100) == -2             # seq_len not a multiple of 64
    assert call(S=0) == -2
    assert call(D=128) == -3             # head size
    assert call(bm=32, bn=32) == -3      # block size
    assert call(q=P + 2) == -4           # misaligned pointer
    assert call(qs=_s3(12 * 128 * 64, 128 * 64, 65)) == -4   # stride not a multiple of 8
    assert call(lbs=2) == -6             # per-sample LUT stride too small
    assert call(form=3) == -3            # launch form
    assert call(dtype=2) == -3           # element format


def test_attention_plan_argument_checks(lib):
    P = 4096
    # bytes: (query-block groups) x (key blocks + 2 header words, rounded up to 8) x 8 per LUT sample
    assert lib.stof_attn_plan_bytes(4096, 2, 1) == 32 * 72 * 8
    assert lib.stof_attn_plan_bytes(4096, 1, 3) == 3 * 64 * 72 * 8
    assert lib.stof_attn_plan_bytes(192, 2, 1) == 2 * 8 * 8
    assert lib.stof_attn_plan_bytes(65536 + 64, 2, 1) == 0      # beyond the plan's key-block range
    assert lib.stof_attn_plan_bytes(4096, 3, 1) == 0
    assert lib.stof_attn_plan_bytes(100, 2, 1) == 0
    assert lib.stof_attn_plan_build(None, P, P, P, 512, 0, 1, 2, P, 1 << 20, None) == -1
    assert lib.stof_attn_plan_build(P, P, P, P, 512, 0, 1, 2, P, 8, None) == -2          # buffer too small
    assert lib.stof_attn_plan_build(P, P, P, P, 512, 0, 1, 2, P + 4, 1 << 20, None) == -4
    assert lib.stof_attn_plan_build(P, P, P, P, 512, 4, 2, 2, P, 1 << 20, None) == -6     # row-pointer stride too small
    assert lib.stof_attn_plan_build(P, P, P, P, 1 << 20, 0, 1, 2, P, 1 << 30, None) == -3
    assert lib.stof_attn_plan_rows(1, 12, 100, -1) == -2
    assert lib.stof_attn_plan_rows(1, 12, 512, 5) == -3
    assert lib.stof_attn_plan_rows(8, 12, 1024, 0) == 2
    assert lib.stof_attn_plan_rows(8, 12, 1024, 1) == 1
    assert lib.stof_attn_plan_rows(8, 12, 1024, 2) == 0


def test_other_entry_points_argument_checks(lib):
    P = 4096
    assert lib.stof_pack_mask_bits(None, P, 64, 64, 64, 1, None) == -1
    assert lib.stof_pack_mask_bits(P, P, 64, 100, 100, 1, None) == -2
    assert lib.stof_bias_res_ln(P, None, None, None, None, P, None, None, 10, 12, 1e-5, None) == -2   # N % 8
    assert lib.stof_bias_res_ln(P, None, None, None, None, P, None, None, 10, 16384, 1e-5, None) == -2
    assert lib.stof_bias_res_ln(None, None, None, None, None, P, None, None, 10, 64, 1e-5, None) == -1
    assert lib.stof_gemm_bias_act(P, P, None, P, 64, 64, 96, 96, 64, 0, None) == -2      # K % 64
    assert lib.stof_gemm_bias_act(P, P, None, P, 64, 64, 64, 64, 64, 9, None) == -3      # activation
    assert lib.stof_gemm_bias_act(P, P + 8, None, P, 64, 64, 64, 64, 64, 0, None) == -4
    # split-K form: A, Wt, bias, C, M, N, K, lda, ldc, act, splits, workspace, bytes, stream
    assert lib.stof_gemm_bias_act_splitk_plan(512, 768, 3072) == 3       # 48 tiles of 64 x 128, 96 k-tiles
    assert lib.stof_gemm_bias_act_splitk_plan(1024, 768, 3072) == 2      # 96 tiles: two splits stay within 256 workgroups
    assert lib.stof_gemm_bias_act_splitk_plan(512, 768, 768) == 1        # 24 k-tiles: too short to split
    assert lib.stof_gemm_bias_act_splitk_plan(2048, 768, 3072) == 1      # 192 tiles already
    assert lib.stof_gemm_bias_act_splitk_plan(8192, 3072, 768) == 1 and lib.stof_gemm_bias_act_splitk_plan(512, 768, 100) == 1
    assert lib.stof_gemm_bias_act_splitk_plan(4096, 768, 3072) == 2      # 192 tiles of 128 x 128 on 256 compute units, long K
    assert lib.stof_gemm_bias_act_splitk_plan(4096, 768, 768) == 1 and lib.stof_gemm_bias_act_splitk_plan(8192, 768, 3072) == 1
    sneed = lib.stof_gemm_bias_act_splitk_workspace_bytes(512, 768, 4)
    assert sneed == 4096 * 16 + 24 * 4 * 128 * 128 * 4      # counters, then 4 splits of 4 x 6 tiles of 128 x 128 floats
    assert lib.stof_gemm_bias_act_splitk_workspace_bytes(512, 768, 9) == 0 and lib.stof_gemm_bias_act_splitk_workspace_bytes(1 << 20, 768, 2) == 0
    sk = lambda **kw: lib.stof_gemm_bias_act_splitk(kw.get("A", P), P, None, P, kw.get("M", 512), 768, kw.get("K", 3072), 3072, 768,
                                                    kw.get("act", 0), kw.get("splits", 4), kw.get("ws", P), kw.get("wsb", sneed), None)
    assert sk(ws=None) == -1
    assert sk(K=3088) == -2 and sk(splits=1) == -2 and sk(splits=9) == -2
    assert sk(wsb=sneed - 1) == -2         # workspace too small
    assert sk(act=9) == -3 and sk(M=1 << 20, wsb=1 << 40) == -3      # more tiles than the counter area holds
    assert sk(A=P + 8) == -4 and sk(ws=P + 8) == -4
    # the entry points that take the element format: 0 fp16, 1 bfloat16, anything else unsupported
    assert lib.stof_gemm_bias_act_dt(P, P, None, P, 64, 64, 64, 64, 64, 0, 2, None) == -3
    assert lib.stof_gemm_bias_act_dt(P, P, None, P, 64, 64, 96, 96, 64, 0, 1, None) == -2      # K % 64, as without the suffix
    assert lib.stof_bias_res_ln_dt(P, None, None, None, None, P, None, None, 10, 64, 1e-5, 7, None) == -3
    assert lib.stof_gemm_bias_act_splitk_dt(P, P, None, P, 512, 768, 3072, 3072, 768, 0, 4, P, sneed, 2, None) == -3
    assert lib.stof_gemm_bias_res_ln_cluster_dt(P, P, None, None, None, None, P, 8192, 768, 768, 768, 768, 768, 1e-5, P, 1 << 30, 5, None) == -3
    # chained GEMM + activation + GEMM: X, W1t, b1, W2t, b2, Y, M, K, F, H, ldx, ldy, act, workspace, bytes, stream
    need = lib.stof_gemm_act_gemm_workspace_bytes(64, 128)
    assert need >= 64 * 128 * 4 + 4 and lib.stof_gemm_act_gemm_workspace_bytes(0, 128) == 0
    chain = lambda **kw: lib.stof_gemm_act_gemm(kw.get("X", P), P, None, P, None, P, 64, kw.get("K", 64), kw.get("F", 128),
                                                kw.get("H", 128), 64, 128, kw.get("act", 1), kw.get("ws", P),
                                                kw.get("wsb", need), None)
    assert chain(ws=None) == -1
    assert chain(K=96) == -2 and chain(F=192) == -2 and chain(H=64) == -2
    assert chain(wsb=need - 1) == -2       # workspace too small
    assert chain(act=9) == -3
    assert chain(X=P + 8) == -4
    assert lib.stof_gemm_bias_res_ln(P, P, None, None, None, None, P, 64, 384, 64, 1e-5, None) == -3   # N
    assert lib.stof_gemm_bias_res_ln(P, P, None, None, None, None, P, 64, 768, 48, 1e-5, None) == -2   # K % 32
    # cluster form: A, Wt, bias, residual, gamma, beta, C, M, N, K, lda, ldr, ldc, eps, workspace, bytes, stream
    cneed = lib.stof_gemm_bias_res_ln_cluster_workspace_bytes(8192, 768)
    assert cneed >= 64 * 12 * 128 * 8 and cneed % 256 == 0
    assert lib.stof_gemm_bias_res_ln_cluster_workspace_bytes(8192, 384) == 8192 // 128 * 6 * 1024 + lib.stof_gemm_bias_res_ln_cluster_workspace_bytes(128, 128) - 2048
    assert lib.stof_gemm_bias_res_ln_cluster_workspace_bytes(8192, 100) == 0          # N % 128
    assert lib.stof_gemm_bias_res_ln_cluster_workspace_bytes((1 << 21) + 1, 768) == 0   # more rows than the counter area holds
    cl = lambda **kw: lib.stof_gemm_bias_res_ln_cluster(kw.get("A", P), P, None, kw.get("res", None), None, None, P, kw.get("M", 8192),
                                                        kw.get("N", 768), kw.get("K", 768), kw.get("lda", 768), kw.get("ldr", 768), kw.get("ldc", 768), 1e-5,
                                                        kw.get("ws", P), kw.get("wsb", cneed), None)
    assert cl(ws=None) == -1
    assert cl(K=96) == -2 and cl(lda=512) == -2 and cl(M=(1 << 21) + 1) == -2
    assert cl(wsb=cneed - 1) == -2          # workspace too small
    assert cl(N=320) == -3 and cl(N=128) == -3 and cl(N=2048, ldc=2048) == -3      # multiples of 128 from 256 to 1024
    assert cl(A=P + 8) == -4 and cl(res=P + 8) == -4 and cl(res=P, ldr=772) == -4
    assert lib.stof_rowwise_attn_fwd(P, P, P, P, 7, 0, 0, None, 1, 128, 12, 64, 0, -1, None) == -3
    assert lib.stof_rowwise_attn_fwd(P, P, P, P, 2, 0, 0, None, 1, 128, 12, 64, 0, -1, None) == -1            # mask kind, no bits
    assert lib.stof_rowwise_attn_fwd(P, P, P, P, 1, 1, 0, None, 1, 128, 12, 64, 0, -1, None) == -2            # band <= 0
    assert lib.stof_rowwise_attn_fwd(P, P, P, P, 0, 0, 0, None, 1, 130, 12, 64, 0, -1, None) == -2
    assert lib.stof_rowwise_attn_fwd(P, P, P, P, 0, 0, 0, None, 1, 128, 12, 64, 0, 5, None) == -3           # launch form


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.StofError):
        _lib.lib()


def test_lut_build_argument_checks(lib):
    P = 4096
    i = lambda **kw: lib.stof_build_lut(kw.get("mask", P), kw.get("eb", 2), kw.get("ld", 256), kw.get("S", 256), kw.get("bm", 64), kw.get("bn", 64),
                                        P, P, P, P, P, P, kw.get("bits", None), None, 16, 16, 16, kw.get("ws", P), kw.get("wsb", 1 << 20), None)
    assert i(mask=None) == -1
    assert i(eb=1) == -3                       # element size
    assert i(bm=48) == -3                      # block size
    assert i(S=200) == -2                      # not divisible
    assert i(ld=128) == -2                     # pitch below S
    assert i(ld=257) == -4                     # rows not 16-byte aligned
    assert i(bits=P, bm=32, bn=32) == -3       # bit rows exist for 64 x 64 only
    assert i(ws=None) == -1
    assert i(wsb=100) == -2                    # workspace too small
    # class bytes (a multiple of 256) + 512 B of bit rows per 64 x 64 tile + 2 B of count per tile (a multiple of 16) + 16
    assert lib.stof_build_lut_workspace_bytes(4096, 64, 64) == 4096 + 4096 * 512 + 4096 * 2 + 16
    assert lib.stof_build_lut_workspace_bytes(256, 16, 16) == 256 + 256 * 2 + 16
    assert lib.stof_build_lut_nnz_offset(256, 16, 16) == 256 + 256 * 2
    assert lib.stof_lut_additive_blocks(P, 2, 256, 256, 64, 64, None, None, 0, None, None) == 0
    assert lib.stof_lut_additive_blocks(P, 2, 256, 256, 64, 64, None, None, 3, None, None) == -1
