"""CPU oracle: masked multi-head attention.

TEST INFRASTRUCTURE ONLY - never imported by the shipped package.

* ``torch_attn_std``       restates src/benchmk_attn_unified.py:20-30, the dense
                           PyTorch-native attention every reference kernel is
                           compared with (src/correct_verify_attn.py:19-30).
                           This is also the function the CPU baseline times.
* ``block_attn_mask``      restates the LUT-driven online-softmax algorithm of the
                           reference block kernel
                           (src/ops/src/block_attn_mask_cuda.cu:3526-3799 with the
                           softmax helper at :183-222) in float arithmetic.
* ``rowwise_attn_*``       restate src/ops/src/rowwise_attn_{full,sliding,mask}_cuda.cu
                           (dense/causal, window, element mask; output [B,S,H*D]).

Rows of the mask with no allowed key are a don't-care in the reference (the
dense path returns a softmax over the raw scores, the block kernel divides by an
uninitialised sum); this oracle DEFINES them as zero output and reports them via
``valid_rows`` so that tests can exclude or pin them.

Pins (tests/test_oracle_attention.py): F.scaled_dot_product_attention with a
boolean mask (library routine), float64 brute force on tiny shapes, all-full LUT
== dense, causal LUT == is_causal, key-block permutation invariance, V == 1
gives rows of ones.
"""
import math

import numpy as np
import torch

NEG_MASK = -10000.0


def torch_attn_std(q, k, v, mask=None):
    """src/benchmk_attn_unified.py:20-30. q,k,v [B,H,S,D]; mask [B,S,S] of 0/1."""
    scores = torch.matmul(q, k.transpose(-2, -1))
    scores = scores / (q.shape[-1] ** .5)
    if mask is not None:
        scores = scores - 10000.0 * (1.0 - mask.unsqueeze(1).to(scores.dtype))
    probs = torch.nn.functional.softmax(scores, dim=-1)
    return torch.matmul(probs, v)


def valid_rows(mask):
    """[B,S] bool: query rows that have at least one allowed key."""
    return (torch.as_tensor(mask) != 0).any(dim=-1)


def dense_masked_attention(q, k, v, mask, dtype=torch.float32):
    """Dense reference with the zero-row definition: torch_attn_std in ``dtype``
    and rows without any allowed key forced to zero."""
    mask = torch.as_tensor(mask)
    if mask.dim() == 2:
        mask = mask.unsqueeze(0)
    mask = mask.expand(q.shape[0], -1, -1)
    out = torch_attn_std(q.to(dtype), k.to(dtype), v.to(dtype), mask.to(dtype))
    ok = valid_rows(mask)  # [B,S]
    return out * ok[:, None, :, None].to(dtype)


def block_attn_mask(q, k, v, lut, block_m, block_n, dtype=np.float32):
    """LUT-driven attention, src/ops/src/block_attn_mask_cuda.cu:3606-3798.

    q,k,v: numpy [B,H,S,D]. ``lut`` is the 8-tuple of get_sparse_storage (shared
    by every batch and head, as in the reference).  Per query block, key blocks
    are visited in LOAD order; a block found next in the FULL list adds nothing,
    one found next in the PARTIAL list adds its additive mask block before the
    scale is applied (:3695 then :193); running max / sum / output follow
    :183-222 and :3755-3757; the output is divided by the running sum (:3794).
    Returns a new array (the reference overwrites q).
    """
    _, frp, fci, prp, pci, pbm, lrp, lci = lut
    B, H, S, D = q.shape
    scale = dtype(1.0 / math.sqrt(D))
    out = np.zeros((B, H, S, D), dtype=dtype)
    q = q.astype(dtype); k = k.astype(dtype); v = v.astype(dtype)
    for r in range(S // block_m):
        rows = slice(r * block_m, (r + 1) * block_m)
        m_run = np.full((B, H, block_m), -np.inf, dtype=dtype)
        l_run = np.zeros((B, H, block_m), dtype=dtype)
        acc = np.zeros((B, H, block_m, D), dtype=dtype)
        fi, pi = frp[r], prp[r]
        for t in range(lrp[r], lrp[r + 1]):
            c = lci[t]
            cols = slice(c * block_n, (c + 1) * block_n)
            s = np.einsum('bhmd,bhnd->bhmn', q[:, :, rows], k[:, :, cols])
            if fi < frp[r + 1] and fci[fi] == c:
                fi += 1
            elif pi < prp[r + 1] and pci[pi] == c:
                s = s + pbm[pi].astype(dtype)[None, None]
                pi += 1
            else:
                continue
            s = s * scale
            m_new = np.maximum(m_run, s.max(-1))
            p = np.exp(s - m_new[..., None])
            alpha = np.exp(m_run - m_new)
            l_run = l_run * alpha + p.sum(-1)
            acc = acc * alpha[..., None] + np.einsum('bhmn,bhnd->bhmd', p, v[:, :, cols])
            m_run = m_new
        with np.errstate(invalid='ignore', divide='ignore'):
            o = acc / l_run[..., None]
        # Zero-row definition: a row whose running max never rose above the
        # additive mask level saw no allowed key.
        dead = ~(m_run > dtype(NEG_MASK * scale * 0.5))
        o[dead] = 0
        out[:, :, rows] = o
    return out


def _merge_heads(o):
    """[B,H,S,D] -> [B,S,H*D], the result layout of the row-wise ops
    (src/ops/package_op.py:13-17)."""
    B, H, S, D = o.shape
    return o.permute(0, 2, 1, 3).reshape(B, S, H * D)


def _rowwise(q, k, v, allowed, dtype):
    """softmax over the allowed keys only; ``allowed`` [S,S] bool."""
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    scores = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(q.shape[-1])
    scores = scores.masked_fill(~allowed[None, None], float('-inf'))
    any_ok = allowed.any(-1)
    probs = torch.softmax(scores, dim=-1)
    probs = torch.where(any_ok[None, None, :, None], probs, torch.zeros_like(probs))
    return _merge_heads(torch.matmul(probs, v))


def rowwise_attn_full(q, k, v, is_causal=False, dtype=torch.float32):
    """src/ops/src/rowwise_attn_full_cuda.cu:20-136: keys 0..(causal ? row : S-1)."""
    S = q.shape[2]
    i = torch.arange(S)[:, None]; j = torch.arange(S)[None, :]
    allowed = (j <= i) if is_causal else torch.ones(S, S, dtype=torch.bool)
    return _rowwise(q, k, v, allowed, dtype)


def rowwise_attn_sliding(q, k, v, is_causal, bandwidth, dtype=torch.float32):
    """src/ops/src/rowwise_attn_sliding_cuda.cu:14-71: row-band < col <= right bound."""
    S = q.shape[2]
    i = torch.arange(S)[:, None]; j = torch.arange(S)[None, :]
    allowed = j > i - bandwidth
    if is_causal:
        allowed = allowed & (j <= i)
    return _rowwise(q, k, v, allowed, dtype)


def rowwise_attn_mask(q, k, v, is_causal, row_mask, dtype=torch.float32):
    """src/ops/src/rowwise_attn_mask_cuda.cu:31-86: row_mask[S,S] > 0, and col <= row
    when causal."""
    S = q.shape[2]
    i = torch.arange(S)[:, None]; j = torch.arange(S)[None, :]
    allowed = torch.as_tensor(row_mask).float() > 0
    if is_causal:
        allowed = allowed & (j <= i)
    return _rowwise(q, k, v, allowed, dtype)
