"""Build libstof_hip.so: every .hip file of this directory, compiled for gfx950 with hipcc
and linked into one shared library placed next to the Python loader (stof/libstof_hip.so).

Usage:  python csrc/build.py
The library has a plain C ABI (include/stof_abi.h); it links against the HIP runtime only.
Then the pybind11 module stof/_stof_ext (csrc/stof_ext.cpp, g++), the Python binding of that ABI.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(os.path.dirname(HERE), "stof", "libstof_hip.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators live in VGPRs: no v_accvgpr copies around the softmax / epilogues
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-I" + os.path.join(ROOT, "include"), "-I" + HERE,
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith(".hip"))


def build(force=True, verbose=True):
    srcs = sources()
    deps = srcs + [os.path.join(HERE, "stof_common.h"), os.path.join(ROOT, "include", "stof_abi.h")]
    if not force and os.path.exists(OUT) and all(os.path.getmtime(OUT) >= os.path.getmtime(d) for d in deps):
        return OUT
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + srcs + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    return OUT


def build_ext(verbose=True):
    """The pybind11 module stof/_stof_ext<suffix>: csrc/stof_ext.cpp, host compiler only, linked
    against libstof_hip.so (run path $ORIGIN).  Returns its path, or None where pybind11 is not
    installed (the ctypes binding serves then)."""
    import sysconfig
    try:
        import pybind11
    except ImportError:
        return None
    out = os.path.join(os.path.dirname(OUT), "_stof_ext" + sysconfig.get_config_var("EXT_SUFFIX"))
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
           "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(ROOT, "include"),
           os.path.join(HERE, "stof_ext.cpp"), "-o", out, "-L" + os.path.dirname(OUT), "-lstof_hip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the extension module failed:\n" + r.stderr)
    return out


if __name__ == "__main__":
    print(build(force=True))
    print(build_ext())
