"""CPU oracle: fused encoder operators and the post-LayerNorm encoder layer.

TEST INFRASTRUCTURE ONLY - never imported by the shipped package.

Restates, in plain PyTorch on the CPU:

* ``matmul_bias_layernorm``   src/triton_template/gemm_add_layernorm.py:78-144
                              (LayerNorm of A@B + bias with NO gamma/beta)
* ``batched_bias_layernorm``  src/triton_template/add_layernorm.py:19-107
* ``matmul_gelu_matmul``      src/triton_template/gemm_gemm.py:99-174 (tanh GELU)
* ``new_gelu``                src/benchmk_end2end.py:25-26
* ``bert_layer``              the torch_attention branch of bert_fwd_std,
                              src/benchmk_end2end.py:31-88, preceded by the QKV
                              projection of src/model-candidate/1-BERT-large.py:17-18
                              when a QKV weight is given.

Pins (tests/test_oracle_encoder.py): F.layer_norm / F.gelu as library routines,
closed forms (zero mean, unit variance for gamma=1 beta=0; W = I; zero residual)
and a float64 re-evaluation.
"""
import math

import torch
import torch.nn.functional as F

from .attention import dense_masked_attention


def _r16(t, on):
    """Round to fp16 and back: where the fp16 eager path of the reference (every tensor of
    src/benchmk_end2end.py:31-88 is fp16 on the GPU) and the five kernels of the product store
    a tensor between two operators."""
    return t.to(torch.float16).to(t.dtype) if on else t


def new_gelu(x):
    """src/benchmk_end2end.py:25-26 (tanh approximation)."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))


def layer_norm(x, gamma=None, beta=None, eps=1e-5):
    """mean / biased variance over the last dim, as both Triton kernels compute it
    (gemm_add_layernorm.py:114-120, add_layernorm.py:44-61)."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps)
    if gamma is not None:
        y = y * gamma
    if beta is not None:
        y = y + beta
    return y


def matmul_bias_layernorm(A, B, bias, eps=1e-5, dtype=torch.float32):
    """src/triton_template/gemm_add_layernorm.py:126-144.

    A [b,M,K], B [b,K,N]; LayerNorm without affine of A@B + bias.  The reference
    kernel reads ``bias[0:N]`` only (:112); its only caller passes
    ``bias + residual`` of shape [b,M,N] (src/tuning_STOF_cost.py:60), so the
    evident intent - a per-element addend - is what this oracle defines: ``bias``
    broadcasts against [b,M,N].
    """
    c = torch.matmul(A.to(dtype), B.to(dtype)) + bias.to(dtype)
    return layer_norm(c, eps=eps)


def batched_bias_layernorm(x, bias, weight, bias_ln, eps=1e-5, dtype=torch.float32):
    """src/triton_template/add_layernorm.py:86-107: LN(x + bias) * weight + bias_ln."""
    return layer_norm(x.to(dtype) + bias.to(dtype), weight.to(dtype), bias_ln.to(dtype), eps)


def matmul_gelu_matmul(a, b, d, bias, dtype=torch.float32):
    """src/triton_template/gemm_gemm.py:158-174: gelu_tanh(a@b + bias) @ d, with the
    intermediate rounded to fp16 before the second product (:152)."""
    t = new_gelu(torch.matmul(a.to(dtype), b.to(dtype)) + bias.to(dtype))
    t = t.to(torch.float16).to(dtype)
    return torch.matmul(t, d.to(dtype))


def gemm_bias_act(x, W, bias, act="none", dtype=torch.float32):
    """x@W + bias followed by none | gelu (erf, F.gelu default as at
    src/benchmk_end2end.py:81) | gelu_tanh (new_gelu) | relu (T5, :206)."""
    y = torch.matmul(x.to(dtype), W.to(dtype)) + bias.to(dtype)
    if act == "gelu":
        return F.gelu(y)
    if act == "gelu_tanh":
        return new_gelu(y)
    if act == "relu":
        return torch.relu(y)
    assert act == "none"
    return y


def gemm_bias_residual_layernorm(x, W, bias, residual, gamma, beta, eps=1e-5, dtype=torch.float32, round_product=False):
    """src/benchmk_end2end.py:73-76 / :83-86: LN(x@W + bias + residual; gamma, beta).
    ``round_product`` rounds x@W to fp16 first, as the reference's fp16 ``torch.matmul`` does
    (:73, :83) and as a GEMM kernel followed by a separate LayerNorm kernel does."""
    y = _r16(torch.matmul(x.to(dtype), W.to(dtype)), round_product) + bias.to(dtype) + residual.to(dtype)
    return layer_norm(y, gamma.to(dtype), beta.to(dtype), eps)


def transpose_for_scores(x, n_heads, head_size):
    """src/util/utils.py:30-34: [B,S,H*D] -> [B,H,S,D]."""
    return x.view(x.shape[:-1] + (n_heads, head_size)).permute(0, 2, 1, 3)


def bert_layer(x, p, mask, n_heads, eps=1e-5, gelu="erf", dtype=torch.float32, round_fp16=False):
    """One post-LayerNorm encoder layer, src/benchmk_end2end.py:31-88.

    ``round_fp16=True`` rounds the tensors that cross an operator boundary (qkv, the attention
    result, the first LayerNorm's output, the FFN activation, the layer output) to fp16, as
    the reference's fp16 eager layer does at the same points; all arithmetic inside an
    operator stays in ``dtype``.  ``round_fp16="split"`` additionally rounds the two products
    that feed a LayerNorm (the eager layer's fp16 matmul outputs, :73 and :83); a pair of flags
    ``(attention-output product, FFN-output product)`` rounds only the ones named.  ``gelu``: "erf" (:81), "tanh" (new_gelu, :25-26) or "relu" (:206).

    ``p`` is a dict of weights in the reference's [in, out] orientation:
    W_qkv [D,3D] (or None: then p['qkv_act'] [B,S,3D] plays the reference's
    pre-made activation, :37), b_qkv, W_o, b_o, g1, be1, W_1, b_1, W_2, b_2, g2, be2.
    ``mask`` [B,S,S] of 0/1.  Rows without an allowed key attend to nothing
    (zero context vector), the oracle's definition for don't-care rows.
    """
    x = x.to(dtype)
    D = x.shape[-1]
    hd = D // n_heads
    if p.get("W_qkv") is not None:
        qkv = torch.matmul(x, p["W_qkv"].to(dtype)) + p["b_qkv"].to(dtype)
    else:
        qkv = p["qkv_act"].to(dtype) + p["b_qkv"].to(dtype)
    rp_o = rp_2 = round_fp16 == "split"
    if isinstance(round_fp16, tuple):
        rp_o, rp_2 = bool(round_fp16[0]), bool(round_fp16[1])
        round_fp16 = True
    qkv = _r16(qkv, round_fp16)
    q, k, v = qkv.chunk(3, dim=-1)
    q = transpose_for_scores(q, n_heads, hd)
    k = transpose_for_scores(k, n_heads, hd)
    v = transpose_for_scores(v, n_heads, hd)
    h = dense_masked_attention(q, k, v, mask, dtype)
    h = _r16(h.permute(0, 2, 1, 3).contiguous().view(x.shape), round_fp16)
    h = _r16(gemm_bias_residual_layernorm(h, p["W_o"], p["b_o"], x, p["g1"], p["be1"], eps, dtype, rp_o), round_fp16)
    r = h
    act = {"erf": "gelu", "tanh": "gelu_tanh", "relu": "relu"}[gelu]
    h = _r16(gemm_bias_act(h, p["W_1"], p["b_1"], act, dtype), round_fp16)
    return _r16(gemm_bias_residual_layernorm(h, p["W_2"], p["b_2"], r, p["g2"], p["be2"], eps, dtype, rp_2), round_fp16)
