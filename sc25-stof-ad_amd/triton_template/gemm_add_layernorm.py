"""Import path of the reference's fused GEMM + bias + LayerNorm template
(src/triton_template/gemm_add_layernorm.py:126-144), served by the HIP MFMA kernel."""
from stof.fused import triton_matmul_bias_layernorm  # noqa: F401
