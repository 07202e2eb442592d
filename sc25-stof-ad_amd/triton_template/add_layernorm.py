"""Import path of the reference's bias + LayerNorm template
(src/triton_template/add_layernorm.py:86-107), served by the HIP kernel."""
from stof.fused import triton_batched_bias_layernorm  # noqa: F401
