"""Binding of libstof_hip.so (C ABI declared in include/stof_abi.h).

Two bindings of the same functions, same names, same positional arguments:
  * the extension module ``_stof_ext`` (pybind11, built by csrc/build.py next to the library;
    the counterpart of the reference's pybind11 modules, src/ops/src/block_attn_mask.cpp:52-56):
    pointers and the stream are ints, None is NULL, a stride triple is a tuple of three ints;
  * ctypes on the library itself, used when the extension module is absent (no pybind11 at
    build time) or when ``STOF_BINDING=ctypes`` is set.
``lib()`` returns whichever is in use; ``i64x3`` builds a stride triple for it.

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
    "stof_device_compute_units": (c_int, []),
    "stof_probe_clock": (c_int, [_P, c_int, _P]),
    "stof_probe_issue_mix": (c_int, [c_int, c_int, c_int, _P, _P, _P]),
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
    "stof_pack_mask_bits": (c_int, [_P, _P, c_int64, c_int64, c_int64, c_int, _P]),
    "stof_rowwise_attn_fwd": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, _P,
                                      c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "stof_build_lut_workspace_bytes": (c_int64, [c_int, c_int, c_int]),
    "stof_build_lut_nnz_offset": (c_int64, [c_int, c_int, c_int]),
    "stof_build_lut": (c_int, [_P, c_int, c_int64, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P,
                               c_int64, c_int64, c_int64, _P, c_int64, _P]),
    "stof_retile_lut": (c_int, [_P, _P, _P, _P, _P, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P,
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
    "stof_gemm_bias_res_ln_cluster_bounded": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                      c_float, _P, c_int64, c_int, c_int, _P]),
    "stof_gemm_bias_res_ln_cluster": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                              c_float, _P, c_int64, _P]),
}


class StofError(RuntimeError):
    """A C-ABI call returned a negative status."""


_ext_used = False


def _load_ctypes():
    h = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(h, name)
        fn.restype = res
        fn.argtypes = args
    return h


def _load_ext():
    """The extension module, or None if it is not built or is older than the library."""
    import importlib.util
    import sysconfig
    path = os.path.join(os.path.dirname(LIB_PATH), "_stof_ext" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))
    if not os.path.exists(path) or os.path.getmtime(path) + 1 < os.path.getmtime(LIB_PATH):
        return None
    # the module is linked against libstof_hip.so with an $ORIGIN run path; loading the library
    # first (globally) makes the process use the one at LIB_PATH whatever the loader would find
    ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    spec = importlib.util.spec_from_file_location("_stof_ext", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    if any(not hasattr(mod, name) for name in _SIGNATURES):
        return None
    return mod


def lib(binding=None):
    """Load (once) and return the binding in use; raise if the library is absent.
    ``binding="ctypes"`` / ``"ext"`` returns that binding without changing the one in use."""
    global _lib, _ext_used
    if _lib is not None and binding is None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise StofError(
            f"{LIB_PATH} is missing: build it with `python sc25-stof-ad_amd/csrc/build.py` "
            "(hipcc, gfx950). There is no fallback path.")
    if binding == "ctypes":
        return _load_ctypes()
    if binding == "ext":
        return _load_ext()
    if _lib is None:
        ext = None if os.environ.get("STOF_BINDING", "") == "ctypes" else _load_ext()
        _ext_used = ext is not None
        _lib = ext if ext is not None else _load_ctypes()
    return _lib


def binding_name():
    """"ext" (pybind11 module) or "ctypes": which binding ``lib()`` hands out."""
    lib()
    return "ext" if _ext_used else "ctypes"


def i64x3(a, b, c):
    """An int64[3] argument (the stride triples of the attention entry points) for the binding in use."""
    if _lib is None:
        lib()
    return (a, b, c) if _ext_used else _I64x3(a, b, c)


def check(status, what):
    if status != 0:
        msg = lib().stof_status_string(status).decode()
        raise StofError(f"{what}: {msg} (status {status})")


def strides3(t):
    """(batch, head, seq) element strides of a [B,H,S,D] view as an int64[3]."""
    s = t.stride()
    return i64x3(s[0], s[1], s[2])
