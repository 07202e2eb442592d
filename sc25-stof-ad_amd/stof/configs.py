"""The five benchmark workloads as seeded synthetic inputs.

C1  single block-masked MHA, B1 H12 S512 D64 (fp32 on the CPU reference path):
    causal window of 128 tokens plus the first 64 tokens global, block 64.
C2  block-masked MHA fp16, B8 H12 S1024 D64: banded window of 3 blocks of 64, 2 global
    blocks and 3 random key blocks per query-block row (BigBird style).
C3  BERT-base encoder layer fp16, B16 S512, hidden 768, FFN 3072, eps 1e-12; per-sample
    lengths uniform in [128, 512], key padding combined with a sliding window of 256.
C4  long-sequence MHA fp16, B2 H16 S4096 D64: causal sliding window of 512 plus every
    4th key block (dilated), block 64.
C5  24-layer encoder stack fp16, hidden 1024, 16 heads, FFN 4096, B4 S2048: causal local
    window of 256 plus one global block.

Masks are integer predicates on (query i, key j); tensors come from a seeded
torch.Generator on the CPU (so CPU and GPU runs see the same numbers) and are moved to
the requested device.
"""
import random
from dataclasses import dataclass

import torch

BLOCK = 64


@dataclass(frozen=True)
class AttnConfig:
    name: str
    batch: int
    heads: int
    seq: int
    head_dim: int = 64


@dataclass(frozen=True)
class LayerConfig:
    name: str
    batch: int
    seq: int
    hidden: int
    heads: int
    ffn: int
    layers: int
    eps: float = 1e-12


C1 = AttnConfig("C1", 1, 12, 512)
C2 = AttnConfig("C2", 8, 12, 1024)
C3 = LayerConfig("C3", 16, 512, 768, 12, 3072, 1)
C4 = AttnConfig("C4", 2, 16, 4096)
C5 = LayerConfig("C5", 4, 2048, 1024, 16, 4096, 24)


def _ij(s):
    i = torch.arange(s)[:, None]
    j = torch.arange(s)[None, :]
    return i, j


def mask_c1(s=512):
    i, j = _ij(s)
    return (((i - j) >= 0) & ((i - j) < 128)) | (j < 64) | (i < 64)


def mask_c2(s=1024):
    n = s // BLOCK
    blk = torch.zeros(n, n, dtype=torch.bool)
    for r in range(n):
        for c in range(n):
            if abs(r - c) <= 1 or r < 2 or c < 2:
                blk[r, c] = True
        for c in random.Random(1234 + r).sample(range(n), 3):
            blk[r, c] = True
    return blk.repeat_interleave(BLOCK, 0).repeat_interleave(BLOCK, 1)


def lengths_c3(batch=16, lo=128, hi=512, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (batch,), generator=g)


def mask_c3(batch=16, s=512, window=256, seed=0):
    """[B,S,S] bool: |i-j| <= window and j < L_b."""
    i, j = _ij(s)
    band = (i - j).abs() <= window
    L = lengths_c3(batch, 128, s, seed)
    return band[None] & (j[None] < L[:, None, None]), L


def mask_c4(s=4096):
    i, j = _ij(s)
    c = j // BLOCK
    return (((i - j) >= 0) & ((i - j) < 512)) | ((j <= i) & (c % 4 == 0))


def mask_c5(s=2048):
    i, j = _ij(s)
    return (((i - j) >= 0) & ((i - j) < 256)) | ((j <= i) & (j < 64))


ATTN_MASKS = {"C1": mask_c1, "C2": mask_c2, "C4": mask_c4, "C5": mask_c5}
# Hand-derived (full, partial) block counts at block 64; used as known answers.
BLOCK_COUNTS = {"C1": (21, 12), "C2": (129, 0), "C4": (840, 106), "C5": (118, 59)}


def qkv(cfg, seed=0, dtype=torch.float16, device="cpu", scale=1.0):
    """q, k, v ~ N(0,1) [B,H,S,D] from one seeded CPU generator."""
    g = torch.Generator().manual_seed(seed)
    shape = (cfg.batch, cfg.heads, cfg.seq, cfg.head_dim)
    return tuple((torch.randn(shape, generator=g) * scale).to(dtype).to(device) for _ in range(3))


def layer_weights(hidden, ffn, seed=0, dtype=torch.float16, device="cpu"):
    """Weights ~ N(0, 0.02) in the reference's [in, out] orientation, biases ~ N(0, 0.02),
    gamma = 1 + N(0, 0.02), beta ~ N(0, 0.02)."""
    g = torch.Generator().manual_seed(seed)
    n = lambda *sh: (torch.randn(*sh, generator=g) * 0.02)
    p = {
        "W_qkv": n(hidden, 3 * hidden), "b_qkv": n(3 * hidden),
        "W_o": n(hidden, hidden), "b_o": n(hidden),
        "g1": 1.0 + n(hidden), "be1": n(hidden),
        "W_1": n(hidden, ffn), "b_1": n(ffn),
        "W_2": n(ffn, hidden), "b_2": n(hidden),
        "g2": 1.0 + n(hidden), "be2": n(hidden),
    }
    return {k: v.to(dtype).to(device) for k, v in p.items()}


def layer_input(cfg, seed=1, dtype=torch.float16, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(cfg.batch, cfg.seq, cfg.hidden, generator=g).to(dtype).to(device)
