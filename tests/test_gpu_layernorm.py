"""GPU parity of bias + residual + LayerNorm against the CPU oracle.
Tolerance: |got - want| <= 2e-3 + 1e-2 * |want| (fp16 output vs fp32 oracle)."""
import pytest
import torch

from oracle import encoder as oe
from stof import fused

pytestmark = pytest.mark.gpu


def _close(got, want):
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    assert not bool((err > 2e-3 + 1e-2 * want.abs()).any()), f"max abs err {float(err.max()):.3e}"


@pytest.mark.parametrize("shape,hidden", [((16, 512), 768), ((4, 300), 1024), ((3, 7), 512), ((2, 5), 8), ((1, 9), 4096), ((2, 3), 8192), ((5, 1), 264)])
@pytest.mark.parametrize("eps", [1e-5, 1e-12])
def test_bias_layernorm_matches_oracle(shape, hidden, eps):
    g = torch.Generator().manual_seed(hidden + shape[1])
    x = (torch.randn(*shape, hidden, generator=g) * 2 + 0.5).half()
    bias = torch.randn(hidden, generator=g).half()
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).half()
    b = (0.1 * torch.randn(hidden, generator=g)).half()
    got = fused.triton_batched_bias_layernorm(x.cuda(), bias.cuda(), w.cuda(), b.cuda(), eps)
    _close(got, oe.batched_bias_layernorm(x, bias, w, b, eps))


def test_residual_and_optional_operands():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 768, generator=g).half(); r = torch.randn(64, 768, generator=g).half()
    got = fused.bias_residual_layernorm(x.cuda(), None, r.cuda(), None, None, 1e-5)
    _close(got, oe.layer_norm(x.float() + r.float()))
    mean = got.float().mean(-1); var = got.float().var(-1, unbiased=False)
    assert float(mean.abs().max()) < 2e-3 and float((var - 1).abs().max()) < 1e-2   # closed form
