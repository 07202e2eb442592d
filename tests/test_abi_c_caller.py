"""The boundary as a C or C++ caller sees it: include/stof_abi.h is valid C99 on its own (what cgo,
bindgen or a plain C program would parse), and a C program linked against libstof_hip.so calls
through it - the version, the status strings and the host-side argument checks, which return
before any launch, so no GPU is needed."""
import os
import shutil
import subprocess

import pytest

from stof import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")

C_PROGRAM = r"""
#include <stdio.h>
#include <string.h>
#include "stof_abi.h"

int main(void) {
  int64_t s[3] = {1, 1, 1};
  if (stof_abi_version() != STOF_ABI_VERSION) { printf("version %d != header %d\n", stof_abi_version(), STOF_ABI_VERSION); return 1; }
  if (strcmp(stof_status_string(STOF_OK), stof_status_string(STOF_ERR_BAD_SHAPE)) == 0) { printf("status strings alike\n"); return 2; }
  /* every pointer NULL: rejected on the host, nothing is launched */
  int rc = stof_block_attn_fwd(NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, 64, 64, 0.125f,
                               s, s, s, s, 1, 64, 1, 64, STOF_DTYPE_F16, 0, -1, NULL);
  if (rc != STOF_ERR_NULL_POINTER) { printf("attention with NULL tensors returned %d\n", rc); return 3; }
  rc = stof_gemm_bias_act(NULL, NULL, NULL, NULL, 8, 8, 64, 64, 8, STOF_ACT_NONE, NULL);
  if (rc != STOF_ERR_NULL_POINTER) { printf("GEMM with NULL tensors returned %d\n", rc); return 4; }
  if (stof_attn_plan_bytes(4096, 2, 1) <= 0 || stof_build_lut_workspace_bytes(4096, 64, 64) <= 0) { printf("size queries\n"); return 5; }
  printf("ok abi %d\n", stof_abi_version());
  return 0;
}
"""


def test_header_is_plain_c99(tmp_path):
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "only_header.c"
    src.write_text('#include "stof_abi.h"\nint main(void) { return STOF_ABI_VERSION > 0 ? 0 : 1; }\n')
    r = subprocess.run([cc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", f"-I{INCLUDE}", str(src)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_c_program_links_and_calls_the_library(tmp_path):
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libstof_hip.so not built (python sc25-stof-ad_amd/csrc/build.py)")
    libdir = os.path.dirname(_lib.LIB_PATH)
    src = tmp_path / "caller.c"
    exe = tmp_path / "caller"
    src.write_text(C_PROGRAM)
    r = subprocess.run([cc, "-std=c99", "-Wall", "-Werror", f"-I{INCLUDE}", str(src), "-o", str(exe),
                        f"-L{libdir}", "-lstof_hip", f"-Wl,-rpath,{libdir}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("ok abi")
