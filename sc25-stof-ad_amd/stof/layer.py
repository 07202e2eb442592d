"""Post-LayerNorm encoder layer and stack on the fused HIP operators.

The layer is the reference's ``bert_fwd_std`` (src/benchmk_end2end.py:31-88) with the QKV
projection of src/model-candidate/1-BERT-large.py:17-18 in front, so that a stack of layers
runs end to end on its own hidden state:

    qkv  = x @ W_qkv + b_qkv                      GEMM + bias              -> [B,S,3D]
    attn = block-masked MHA(q, k, v; LUT)          q/k/v read in place from qkv, result [B,S,D]
    h    = LN(attn @ W_o + b_o + x; g1, be1)       GEMM + bias + residual + LayerNorm
    f    = GELU(h @ W_1 + b_1)                     GEMM + bias + GELU
    y    = LN(f @ W_2 + b_2 + h; g2, be2)          GEMM + bias + residual + LayerNorm

Five launches per layer, no permute / contiguous copies, no standalone elementwise kernels.
``ln_fusion`` selects how the two LayerNorm GEMMs run: "fused" = LayerNorm in the GEMM
epilogue with one workgroup owning the full row, "cluster" = LayerNorm in the epilogue of the
128 x 128-tile GEMM, the workgroups of a row block exchanging row statistics, "split" = tiled
GEMM followed by the bias+residual+LayerNorm kernel.  "auto" is a fixed rule on the shape (the
reference likewise switches its fused GEMM+LN per shape, data/triton_perf.csv), not a run-time
tuner.
"""
import torch

from . import fused
from .ops import block_attn, block_attn_packed_qkv


class EncoderLayer:
    def __init__(self, weights, n_heads, eps=1e-12, gelu="erf", ln_fusion="auto", ffn_chain="auto"):
        """``weights``: dict with W_qkv [D,3D], b_qkv, W_o [D,D], b_o, g1, be1, W_1 [D,F], b_1,
        W_2 [F,D], b_2, g2, be2 in the reference's [in, out] orientation, fp16 on the GPU.
        ``ffn_chain``: True / False / "auto" - the two FFN products as one launch with the 4 x hidden
        intermediate on chip (``fused.gemm_act_gemm``); "auto" takes it up to
        ``fused.CHAIN_MAX_ROWS`` rows (0 on MI355X: two launches measured faster at every size)."""
        self.n_heads = n_heads
        self.ffn_chain = ffn_chain
        self.eps = eps
        # FFN activation: erf GELU (BERT, src/benchmk_end2end.py:81), tanh GELU (GPT, :25-26,144), ReLU (T5, :206)
        acts = {"erf": "gelu", "gelu": "gelu", "tanh": "gelu_tanh", "gelu_tanh": "gelu_tanh", "relu": "relu"}
        if gelu not in acts:
            raise ValueError(f"activation must be one of {sorted(acts)}, got {gelu!r}")
        self.act = acts[gelu]
        self.ln_fusion = ln_fusion
        w = weights
        self.Wqkv = w["W_qkv"].t().contiguous(); self.bqkv = w["b_qkv"].contiguous()
        self.Wo = w["W_o"].t().contiguous(); self.bo = w["b_o"].contiguous()
        self.W1 = w["W_1"].t().contiguous(); self.b1 = w["b_1"].contiguous()
        self.W2 = w["W_2"].t().contiguous(); self.b2 = w["b_2"].contiguous()
        self.g1, self.be1 = w["g1"].contiguous(), w["be1"].contiguous()
        self.g2, self.be2 = w["g2"].contiguous(), w["be2"].contiguous()
        self.hidden = self.Wo.shape[0]

    def _ln_form(self, M, K):
        """How a LayerNorm GEMM of M rows and reduction length K runs: "fused" (one workgroup per
        64 rows owns the whole row), "cluster" (128 x 128 tiles, the workgroups of a row block
        exchange row statistics) or "split" (tiled GEMM, then the bias+residual+LayerNorm kernel);
        "auto" follows ``fused.ln_gemm_form``."""
        if self.ln_fusion in ("fused", "cluster", "split"):
            return self.ln_fusion
        return fused.ln_gemm_form(M, self.hidden, K)

    def pre_ln_stored(self, M):
        """For M token rows, whether the product that feeds a LayerNorm is stored as a 16-bit tensor
        first (the split form) or stays in registers (fused and cluster forms): one flag for the
        attention-output GEMM (K = hidden) and one for the FFN-output GEMM (K = ffn) - the two can
        take different forms (4096 rows at hidden 768: cluster for K 768, split-K GEMM + LayerNorm
        kernel for K 3072)."""
        return (self._ln_form(M, self.hidden) == "split", self._ln_form(M, self.W1.shape[0]) == "split")

    def _gemm_ln(self, x, Wt, bias, residual, gamma, beta):
        form = self._ln_form(x.numel() // x.shape[-1], x.shape[-1])
        return fused.gemm_bias_residual_layernorm(x, Wt, bias, residual, gamma, beta, self.eps,
                                                  form="row" if form == "fused" else form)

    def _chain(self, M):
        if self.ffn_chain != "auto":
            return bool(self.ffn_chain)
        return (M <= fused.CHAIN_MAX_ROWS and self._ln_form(M, self.W1.shape[0]) == "split" and
                fused.chain_supported(M, self.hidden, self.W1.shape[0], self.hidden))

    def _ffn(self, h):
        M = h.numel() // h.shape[-1]
        if self._chain(M):
            y = fused.gemm_act_gemm(h, self.W1, self.b1, self.W2, None, self.act)
            return fused.bias_residual_layernorm(y, self.b2, h, self.g2, self.be2, self.eps)
        f = fused.gemm_bias_act(h, self.W1, self.b1, self.act)
        return self._gemm_ln(f, self.W2, self.b2, h, self.g2, self.be2)

    def forward(self, x, lut, block=64, check=False):
        """``check=True`` synchronises the device after the layer and raises if a cluster-form
        LayerNorm GEMM (this layer's or an earlier one on the device) gave up a wait - see
        ``fused.check_cluster_exchange``; for callers that share the device with other work."""
        B, S, D = x.shape
        H = self.n_heads
        hd = D // H
        qkv = fused.gemm_bias_act(x, self.Wqkv, self.bqkv, "none")           # [B,S,3D]
        attn = block_attn_packed_qkv(qkv, H, lut, block, block)               # q, k, v read in place; [B,S,D]
        h = self._gemm_ln(attn, self.Wo, self.bo, x, self.g1, self.be1)
        y = self._ffn(h)
        if check:
            fused.check_cluster_exchange(x.device)
        return y

    __call__ = forward

    def stages(self, x, lut, block=64):
        """The five launches of ``forward`` as (name, thunk) pairs on precomputed inputs, so each
        can be timed on its own (the reference's layer has no QKV projection,
        src/benchmk_end2end.py:37: its figure is the sum without "qkv_gemm")."""
        B, S, D = x.shape
        H = self.n_heads
        hd = D // H
        qkv = fused.gemm_bias_act(x, self.Wqkv, self.bqkv, "none")
        q, k, v = (qkv[..., t * D:(t + 1) * D].view(B, S, H, hd).permute(0, 2, 1, 3) for t in range(3))
        attn = block_attn(q, k, v, lut, block, block, out_layout="bshd")
        h = self._gemm_ln(attn, self.Wo, self.bo, x, self.g1, self.be1)
        f = fused.gemm_bias_act(h, self.W1, self.b1, self.act)
        return [
            ("qkv_gemm", lambda: fused.gemm_bias_act(x, self.Wqkv, self.bqkv, "none")),
            ("attention", lambda: block_attn(q, k, v, lut, block, block, out_layout="bshd")),
            ("out_proj_ln", lambda: self._gemm_ln(attn, self.Wo, self.bo, x, self.g1, self.be1)),
            ("ffn1_gelu", lambda: fused.gemm_bias_act(h, self.W1, self.b1, self.act)),
            ("ffn2_ln", lambda: self._gemm_ln(f, self.W2, self.b2, h, self.g2, self.be2)),
        ]


class EncoderStack:
    """``layers`` independent EncoderLayers applied in sequence (24 for the BERT-large /
    GPT-2-medium style stack)."""

    def __init__(self, layer_weights, n_heads, eps=1e-12, gelu="erf", ln_fusion="auto", ffn_chain="auto"):
        self.layers = [EncoderLayer(w, n_heads, eps, gelu, ln_fusion, ffn_chain) for w in layer_weights]

    def forward(self, x, lut, block=64, check=False):
        """``check=True``: one ``fused.check_cluster_exchange`` after the last layer (it covers all)."""
        for layer in self.layers:
            x = layer(x, lut, block)
        if check:
            fused.check_cluster_exchange(x.device)
        return x

    __call__ = forward


class CapturedForward:
    """A layer or stack recorded once into a HIP graph for one input shape and one LUT and
    replayed from then on: one graph launch instead of five kernel launches per layer.  For
    small batches, where issuing the launches (not running the kernels) sets the pace.

    The constructor runs the module a few times outside the graph first, which also fills the
    per-LUT caches (validation, bit packing), so nothing synchronises or allocates outside
    torch's graph pool while recording.  ``__call__`` copies its argument into the graph's
    input buffer, replays, and returns the graph's output buffer (overwritten by the next call).
    """

    def __init__(self, module, x, lut, block=64, warmup=3):
        self.x = x.clone()
        side = torch.cuda.Stream(device=x.device)
        side.wait_stream(torch.cuda.current_stream(x.device))
        with torch.cuda.stream(side):
            for _ in range(warmup):
                module(self.x, lut, block)
        torch.cuda.current_stream(x.device).wait_stream(side)
        torch.cuda.synchronize(x.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.y = module(self.x, lut, block)

    def __call__(self, x, check=False):
        """``check=True``: synchronise after the replay and raise if a cluster-form LayerNorm GEMM
        gave up a wait (``fused.check_cluster_exchange``)."""
        self.x.copy_(x)
        self.graph.replay()
        if check:
            fused.check_cluster_exchange(self.x.device)
        return self.y


def eager_layer(x, w, mask, n_heads, eps=1e-12, gelu="erf"):
    """The same layer in plain PyTorch ops on x's device (matmul, add, softmax, F.gelu,
    F.layer_norm, permute + contiguous exactly as src/benchmk_end2end.py:31-88): the unfused
    comparator the fused layer is timed against.  ``mask`` [B,S,S] or [1,S,S] of 0/1.
    ``gelu``: "erf" (BERT, :81), "tanh" (GPT, :25-26,144) or "relu" (T5, :206)."""
    import torch.nn.functional as F
    act = {"erf": F.gelu, "tanh": lambda t: F.gelu(t, approximate="tanh"), "relu": F.relu}[gelu]
    B, S, D = x.shape
    hd = D // n_heads
    qkv = torch.matmul(x, w["W_qkv"]) + w["b_qkv"]
    q, k, v = qkv.chunk(3, dim=-1)
    tr = lambda t: t.view(B, S, n_heads, hd).permute(0, 2, 1, 3)
    q, k, v = tr(q), tr(k), tr(v)
    scores = torch.matmul(q, k.transpose(-2, -1)) / (hd ** .5)
    scores -= 10000.0 * (1.0 - mask.unsqueeze(1))
    probs = F.softmax(scores, dim=-1)
    h = torch.matmul(probs, v)
    h = h.permute(0, 2, 1, 3).contiguous().view(B, S, D)
    h = torch.matmul(h, w["W_o"]) + w["b_o"]
    h = F.layer_norm(h + x, (D,), weight=w["g1"], bias=w["be1"], eps=eps)
    r = h
    h = act(torch.matmul(h, w["W_1"]) + w["b_1"])
    h = torch.matmul(h, w["W_2"]) + w["b_2"]
    return F.layer_norm(h + r, (D,), weight=w["g2"], bias=w["be2"], eps=eps)
