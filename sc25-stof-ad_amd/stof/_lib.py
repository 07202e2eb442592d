"""ctypes binding of libstof_hip.so (C ABI declared in include/stof_abi.h).

The library is loaded from this directory.  It is never built implicitly on a machine
with a GPU: a missing library is an error there, so a silent fallback cannot hide it.
"""
import ctypes
import os
from ctypes import c_int, c_int64, c_float, c_void_p, c_char_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libstof_hip.so")

_lib = None

_P = c_void_p
_I64x3 = c_int64 * 3

_SIGNATURES = {
    "stof_abi_version": (c_int, []),
    "stof_status_string": (c_char_p, [c_int]),
    "stof_block_attn_fwd": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,
                                    c_int, c_int, c_float,
                                    POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
                                    c_int, c_int, c_int, c_int, c_int, c_int64, c_int, _P]),
    "stof_block_attn_fwd_planned": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,
                                            c_int, c_int, c_float,
                                            POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
                                            c_int, c_int, c_int, c_int, c_int, c_int64, c_int, _P, c_int64, c_int, _P]),
    "stof_attn_plan_rows": (c_int, [c_int, c_int, c_int, c_int]),
    "stof_attn_plan_bytes": (c_int64, [c_int, c_int, c_int]),
    "stof_attn_plan_build": (c_int, [_P, _P, _P, _P, c_int, c_int64, c_int, c_int, _P, c_int64, _P]),
    "stof_attn_set_launch_form": (c_int, [c_int]),
    "stof_pack_mask_bits": (c_int, [_P, _P, c_int64, c_int64, c_int64, c_int, _P]),
    "stof_rowwise_attn_fwd": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, _P,
                                      c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "stof_build_lut_workspace_bytes": (c_int64, [c_int, c_int, c_int]),
    "stof_build_lut": (c_int, [_P, c_int, c_int64, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P,
                               c_int64, c_int64, c_int64, _P, c_int64, _P]),
    "stof_build_lut_static_max_tiles": (c_int64, []),
    "stof_build_lut_static": (c_int, [_P, c_int, c_int64, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P,
                                      c_int64, c_int64, c_int64, _P]),
    "stof_lut_additive_blocks": (c_int, [_P, c_int, c_int64, c_int, c_int, c_int, _P, _P, c_int64, _P, _P]),
    "stof_bias_res_ln": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_float, _P]),
    "stof_gemm_bias_act": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, _P]),
    "stof_gemm_act_gemm_workspace_bytes": (c_int64, [c_int64, c_int64]),
    "stof_gemm_act_gemm": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                   c_int, _P, c_int64, _P]),
    "stof_gemm_bias_act_splitk_plan": (c_int, [c_int64, c_int64, c_int64]),
    "stof_gemm_bias_act_splitk_workspace_bytes": (c_int64, [c_int64, c_int64, c_int]),
    "stof_gemm_bias_act_splitk": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int,
                                          _P, c_int64, _P]),
    "stof_gemm_bias_res_ln": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_float, _P]),
    "stof_bias_res_ln_dt": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_float, c_int, _P]),
    "stof_gemm_bias_act_dt": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, _P]),
    "stof_gemm_bias_act_splitk_dt": (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int,
                                             _P, c_int64, c_int, _P]),
    "stof_gemm_bias_res_ln_cluster_dt": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                 c_float, _P, c_int64, c_int, _P]),
    "stof_gemm_bias_res_ln_cluster_workspace_bytes": (c_int64, [c_int64, c_int64]),
    "stof_gemm_bias_res_ln_cluster_set_spin_limit": (c_int, [c_int]),
    "stof_gemm_bias_res_ln_cluster": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                              c_float, _P, c_int64, _P]),
}


class StofError(RuntimeError):
    """A C-ABI call returned a negative status."""


def lib():
    """Load (once) and return the ctypes handle; raise if the library is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise StofError(
                f"{LIB_PATH} is missing: build it with `python sc25-stof-ad_amd/csrc/build.py` "
                "(hipcc, gfx950). There is no fallback path.")
        h = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(h, name)
            fn.restype = res
            fn.argtypes = args
        _lib = h
    return _lib


def check(status, what):
    if status != 0:
        msg = lib().stof_status_string(status).decode()
        raise StofError(f"{what}: {msg} (status {status})")


def strides3(t):
    """(batch, head, seq) element strides of a [B,H,S,D] view as an int64[3]."""
    return _I64x3(t.stride(0), t.stride(1), t.stride(2))
