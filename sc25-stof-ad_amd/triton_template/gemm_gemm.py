"""Import path of the reference's chained GEMM + GELU + GEMM template
(src/triton_template/gemm_gemm.py:158-174), served by the HIP MFMA kernels."""
from stof.fused import triton_matmul_batch  # noqa: F401
