"""Masked attention with the reference's module names, one mask family at a time.

The flow is the one of the reference's unified attention benchmark (src/benchmk_attn_unified.py:
build a mask, compile it to the block LUT, let the selector choose an operator, run it, compare
with the dense PyTorch attention): here every import resolves to this package's shims, so the
same lines run on an MI355X.

    python sc25-stof-ad_amd/examples/unified_attention.py --mask bigbird --batch 8 --seq 1024
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from ops.package_op import block_attn_mask_op, rowwise_attn_full_op            # noqa: E402
from util.masks import (generate_bigbird_mask, generate_causal_mask, generate_dilated_mask,  # noqa: E402
                        generate_longformer_mask, generate_sliding_mask, get_sparse_storage)
from util.utils import time_stamp_cudasync, torch_cuda_identify                 # noqa: E402
from stof.selector import GPUParams, apply, select_operator                     # noqa: E402


def dense_attention(q, k, v, mask):
    """softmax(q k^T / sqrt(d) - 10000 (1 - mask)) v in fp32: the check, not the product."""
    s = torch.matmul(q.float(), k.float().transpose(-2, -1)) / q.shape[-1] ** 0.5
    s = s - 10000.0 * (1.0 - mask.unsqueeze(1).float())
    return torch.matmul(torch.softmax(s, dim=-1), v.float())


def build_mask(name, batch, seq, device):
    ones = torch.ones(batch, seq, seq, dtype=torch.float16, device=device)
    if name == "causal":
        return generate_causal_mask(ones)
    if name == "sliding":
        return generate_sliding_mask(ones, bandwidth=seq // 8, is_cauasl=False)
    if name == "dilated":
        return generate_dilated_mask(ones, bandwidth=seq // 8, dilation_rate=1, is_cauasl=False)
    if name == "longformer":
        return generate_longformer_mask(ones, globalwidth=64, bandwidth=seq // 8, is_cauasl=False)
    if name == "bigbird":
        return generate_bigbird_mask(ones, globalwidth=64, bandwidth=seq // 8, fill_rate=0.1, is_cauasl=False)
    raise SystemExit(f"unknown mask {name!r}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--mask", default="bigbird", choices=["causal", "sliding", "dilated", "longformer", "bigbird"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--heads", type=int, default=12)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--iters", type=int, default=200)
    args = ap.parse_args()
    device = torch_cuda_identify(print_info=True)
    if device.type != "cuda":
        raise SystemExit("an MI355X is required: there is no CPU path")
    torch.manual_seed(0)
    shape = (args.batch, args.heads, args.seq, 64)
    q, k, v = (torch.randn(shape, dtype=torch.float16, device=device) for _ in range(3))
    mask = build_mask(args.mask, args.batch, args.seq, device).to(device)   # (the causal generator answers on the CPU, as the reference's does)

    nnz, *lut = get_sparse_storage(mask, 64, 64)          # nnz: the reference's figure, non-zeros of [B,S,S] over S*S in per cent
    active = int(lut[5][-1])                               # last LOAD row pointer = active 64 x 64 blocks
    choice = select_operator(GPUParams("MI355X"), lut[5], args.batch, args.seq, args.heads,
                             is_causal=args.mask == "causal", lut=lut)
    print(f"mask {args.mask}: nnz figure {float(nnz):.1f}, {active} of {(args.seq // 64) ** 2} blocks active; "
          f"selector: {choice} ({choice.reason})")

    want = dense_attention(q, k, v, mask[:1])
    # the selected operator in the selected launch form; [B,S,H*D] like the reference's row-wise operators
    run = lambda: apply(choice, q, k, v, lut, is_causal=args.mask == "causal")
    got = run().view(args.batch, args.seq, args.heads, 64).permute(0, 2, 1, 3)
    # the reference-named operators give the same numbers (the block op writes into its first argument)
    same = block_attn_mask_op(q.clone(), k, v, *lut, 64, 64, 4)
    if args.mask == "causal":
        same = rowwise_attn_full_op(q, k, v, True).view(args.batch, args.seq, args.heads, 64).permute(0, 2, 1, 3)
    assert (same.float() - got.float()).abs().max().item() < 2e-3
    err = (got.float() - want).abs().max().item()
    print(f"max abs difference from dense fp32 attention: {err:.2e}")

    for _ in range(20):
        run()
    t0 = time_stamp_cudasync()
    for _ in range(args.iters):
        run()
    t1 = time_stamp_cudasync()
    flop = 4 * 64 ** 3 * active * args.batch * args.heads
    ms = (t1 - t0) * 1e3 / args.iters
    print(f"{ms * 1e3:.1f} us per call, {flop / ms / 1e9:.0f} TFLOP/s on active blocks")


if __name__ == "__main__":
    main()
