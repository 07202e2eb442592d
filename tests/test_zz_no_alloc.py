"""stof_build_lut_static - the entry point that allocates nothing (its scratch is a fixed array in
device memory) - against stof_build_lut, which takes a caller's workspace: identical outputs, bit
for bit, on two calls in a row, the second with a smaller input."""
import ctypes

import pytest
import torch

from stof import _lib, configs

pytestmark = pytest.mark.gpu


def _outputs(S):
    nq = S // 64
    i32 = lambda n: torch.full((n,), -1, dtype=torch.int32, device="cuda")
    return dict(frp=i32(nq + 1), fci=i32(nq * nq), prp=i32(nq + 1), pci=i32(nq * nq), lrp=i32(nq + 1), lci=i32(nq * nq),
                bits=torch.full((nq * nq, 64), -1, dtype=torch.int64, device="cuda"), counts=i32(4))


def _call(fn, mask, S, o, extra):
    t = S // 64 * (S // 64)
    rc = fn(mask.data_ptr(), mask.element_size(), mask.stride(0), S, 64, 64,
            o["frp"].data_ptr(), o["fci"].data_ptr(), o["prp"].data_ptr(), o["pci"].data_ptr(), o["lrp"].data_ptr(), o["lci"].data_ptr(),
            o["bits"].data_ptr(), o["counts"].data_ptr(), t, t, t, *extra, None)
    assert rc == 0, rc
    torch.cuda.synchronize()


def test_static_scratch_entry_point_matches_workspace_entry_point():
    lib = _lib.lib()
    # first call: C4's mask at S 4096 (840 full + 106 partial tiles); second: C1's at S 512 (21 + 12)
    for name, S, dtype in (("C4", 4096, torch.float16), ("C1", 512, torch.float32)):
        print(f"no-alloc LUT build, case {name} S{S}", flush=True)
        mask = configs.ATTN_MASKS[name](S).to(dtype).cuda()
        a, b = _outputs(S), _outputs(S)
        ws = torch.empty(lib.stof_build_lut_workspace_bytes(S, 64, 64), dtype=torch.uint8, device="cuda")
        _call(lib.stof_build_lut, mask, S, a, (ws.data_ptr(), ws.numel()))
        _call(lib.stof_build_lut_static, mask, S, b, ())
        n_full, n_part, n_load, overflow = a["counts"].tolist()
        assert (n_full, n_part) == configs.BLOCK_COUNTS[name] and not overflow
        assert a["counts"].tolist() == b["counts"].tolist()
        for k, n in (("frp", None), ("prp", None), ("lrp", None), ("fci", n_full), ("pci", n_part), ("lci", n_load), ("bits", n_part)):
            assert torch.equal(a[k][:n], b[k][:n]), f"{name}: {k} differs between the two entry points"
    assert lib.stof_build_lut_static_max_tiles() == 16384
    big = torch.zeros(16, 16, dtype=torch.float16, device="cuda")      # never read: the size check comes first
    o = _outputs(64)
    rc = lib.stof_build_lut_static(big.data_ptr(), 2, 16384, 16384, 64, 64, o["frp"].data_ptr(), o["fci"].data_ptr(), o["prp"].data_ptr(),
                                   o["pci"].data_ptr(), o["lrp"].data_ptr(), o["lci"].data_ptr(), None, None, 1, 1, 1, None)
    assert rc == -7 and b"scratch" in lib.stof_status_string(rc)
