"""Encoder stacks end to end, with the command line of the reference's end-to-end benchmark.

The flow is the one of src/benchmk_end2end.py (:326-545): pick a model (layer count, heads), a
mask family, batch and sequence length; build the mask and compile it to the block LUT; run
the stack with plain PyTorch ops ("TorchNative") and with this library's fused layer ("STOF":
QKV GEMM, block-masked attention, GEMM + bias + residual + LayerNorm, GEMM + bias + activation,
GEMM + bias + residual + LayerNorm); print ms per iteration in the reference's format.  In
addition the two outputs are compared.  T5 is run as its encoder stack (ReLU feed-forward,
:154-210); the decoder's cross attention is not part of this library.

    python sc25-stof-ad_amd/examples/end2end.py --model bert_base --batch_size 8 --seq_len 512 --method both
    python sc25-stof-ad_amd/examples/end2end.py --model gpt --batch_size 1 --seq_len 512 --graph
"""
import argparse
import math
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from util.masks import (generate_bigbird_mask, generate_longformer_mask, generate_sliding_mask,  # noqa: E402
                        get_sparse_storage)
from util.utils import time_stamp_cudasync, torch_cuda_identify                 # noqa: E402
from stof import configs                                                        # noqa: E402
from stof.layer import CapturedForward, EncoderStack, eager_layer               # noqa: E402

# model -> (heads, layers, feed-forward activation); head size 64, hidden = 64 * heads (src/benchmk_end2end.py:383-407)
MODELS = {
    "bert_small": (8, 6, "erf"),
    "bert_base": (12, 12, "erf"),
    "bert_large": (16, 24, "erf"),
    "gpt": (12, 12, "tanh"),
    "t5": (12, 12, "relu"),
}


def build_mask(mask_id, seq, block_m, block_n, device):
    """One [1,S,S] mask of 0/1: 1 sliding, 2 Longformer, 3 BigBird, with the reference's widths
    (global width = BLOCK_M, band width = BLOCK_N, fill rate 0.1; src/benchmk_end2end.py:441-446)."""
    ones = torch.ones(1, seq, seq, dtype=torch.float16, device=device)
    if mask_id == 1:
        return "Sliding_Mask", generate_sliding_mask(ones, bandwidth=block_n, is_cauasl=False)
    if mask_id == 2:
        return "Longformer_Mask", generate_longformer_mask(ones, globalwidth=block_m, bandwidth=block_n, is_cauasl=False)
    if mask_id == 3:
        return "BigBird_Mask", generate_bigbird_mask(ones, globalwidth=block_m, bandwidth=block_n, fill_rate=0.1, is_cauasl=False)
    raise SystemExit("mask_id must be 1 (sliding), 2 (Longformer) or 3 (BigBird)")


def main():
    ap = argparse.ArgumentParser(description="Encoder stack end to end, fused (STOF) against plain PyTorch ops")
    ap.add_argument("--mask_id", type=int, default=3, help="1-Sliding | 2-Longformer | 3-BigBird")
    ap.add_argument("--block_m", type=int, default=64, help="block size of the LUT along the queries")
    ap.add_argument("--block_n", type=int, default=64, help="block size of the LUT along the keys")
    ap.add_argument("--num_warps", type=int, default=4, help="accepted for the reference's command lines; the launch form is chosen by the library")
    ap.add_argument("--method", default="both", choices=["TorchNative", "STOF", "both"])
    ap.add_argument("--model", default="bert_base", choices=sorted(MODELS))
    ap.add_argument("--batch_size", type=int, default=8)
    ap.add_argument("--seq_len", type=int, default=1024)
    ap.add_argument("--graph", action="store_true", help="STOF: record the stack into a HIP graph once and replay it (small batches are paced by issuing the launches)")
    ap.add_argument("--warmup_iters", type=int, default=20)
    ap.add_argument("--running_iters", type=int, default=100)
    args = ap.parse_args()
    device = torch_cuda_identify(print_info=False)
    if device.type != "cuda":
        raise SystemExit("an MI355X is required: there is no CPU path")
    torch.manual_seed(0)
    heads, layers, act = MODELS[args.model]
    hidden, ffn = 64 * heads, 256 * heads
    B, S = args.batch_size, args.seq_len

    mask_name, mask = build_mask(args.mask_id, S, args.block_m, args.block_n, device)
    mask = mask.to(device)
    nnz, *lut = get_sparse_storage(mask, args.block_m, args.block_n)
    print(f"{mask_name}: nnz figure {float(nnz):.1f}, {int(lut[5][-1])} of {math.ceil(S / args.block_m) * math.ceil(S / args.block_n)} blocks active")

    weights = [{k: v.to(device) for k, v in configs.layer_weights(hidden, ffn, seed=100 + i).items()} for i in range(layers)]
    x = configs.layer_input(configs.LayerConfig(args.model, B, S, hidden, heads, ffn, layers), seed=1, device=device)

    def native():
        h = x
        with torch.no_grad():
            for w in weights:
                h = eager_layer(h, w, mask, heads, 1e-12, gelu=act)
        return h

    stack = EncoderStack(weights, heads, eps=1e-12, gelu=act)
    fused = lambda: stack(x, lut, args.block_m)
    if args.graph:
        captured = CapturedForward(stack, x, lut, args.block_m)
        fused = lambda: captured(x)

    def time_ms(fn):
        for _ in range(args.warmup_iters):
            fn()
        t0 = time_stamp_cudasync()
        for _ in range(args.running_iters):
            fn()
        return (time_stamp_cudasync() - t0) * 1000 / args.running_iters

    times = {}
    if args.method in ("TorchNative", "both"):
        times["native"] = time_ms(native)
        print("e2e {} | bs:{} | seq:{}  |  Torch Native    : {:.3f} ms / iter".format(args.model, B, S, times["native"]))
    if args.method in ("STOF", "both"):
        times["stof"] = time_ms(fused)
        print("e2e {} | bs:{} | seq:{}  |  STOF            : {:.3f} ms / iter{}".format(args.model, B, S, times["stof"], " (graph replay)" if args.graph else ""))
    if len(times) == 2:
        print("speedup over Torch Native: {:.2f}x".format(times["native"] / times["stof"]))
    # both paths round to fp16 between their kernels, at different places: the difference grows
    # slowly with depth and stays a small multiple of the fp16 spacing of the O(1) outputs
    err = (fused().float() - native().float()).abs().max().item()
    print(f"max abs difference between the two outputs after {layers} layers: {err:.2e}")


if __name__ == "__main__":
    main()
