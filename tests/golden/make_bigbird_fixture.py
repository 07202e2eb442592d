"""Writes tests/golden/bigbird_ref.npz: outputs of the REFERENCE's own generate_bigbird_mask
(src/util/masks.py:86-122), imported by path from /root/reference in the build container.

Only this function is taken from the running reference: its random part depends on the
exact order of stdlib RNG calls, which no closed form pins.  Every other oracle function is
pinned by closed forms and brute force (tests/test_oracle_masks.py).  The fixture stores
inputs (shape and keyword arguments) and the expected mask as packed bits.

Run once:  python tests/golden/make_bigbird_fixture.py
"""
import importlib.util
import json
import os

import numpy as np
import torch

REF = "/root/reference/src/util/masks.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bigbird_ref.npz")

CASES = [
    dict(batch=1, seq=128, globalwidth=4, bandwidth=2, fill_rate=0.1, is_cauasl=False),
    dict(batch=2, seq=256, globalwidth=32, bandwidth=32, fill_rate=0.1, is_cauasl=False),
    dict(batch=2, seq=192, globalwidth=8, bandwidth=4, fill_rate=0.05, is_cauasl=True),
    dict(batch=1, seq=64, globalwidth=1, bandwidth=1, fill_rate=0.2, is_cauasl=False),
]


def main():
    spec = importlib.util.spec_from_file_location("ref_masks", REF)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    arrays = {"cases": np.frombuffer(json.dumps(CASES).encode(), dtype=np.uint8)}
    for n, c in enumerate(CASES):
        attr = torch.ones(c["batch"], c["seq"], c["seq"], dtype=torch.float16)
        m = ref.generate_bigbird_mask(attr, globalwidth=c["globalwidth"], bandwidth=c["bandwidth"],
                                      fill_rate=c["fill_rate"], is_cauasl=c["is_cauasl"])
        assert set(torch.unique(m).tolist()) <= {0.0, 1.0}
        arrays[f"mask{n}"] = np.packbits(m.numpy().astype(np.uint8).reshape(-1))
    np.savez_compressed(OUT, **arrays)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
