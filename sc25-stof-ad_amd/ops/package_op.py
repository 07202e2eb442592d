"""Import path of the reference's operator module (``from ops.package_op import ...``,
src/ops/package_op.py:7,70-74), served by the HIP implementation."""
from stof.ops import (block_attn_mask_op, rowwise_attn_full_op, rowwise_attn_sliding_op,  # noqa: F401
                      rowwise_attn_mask_op, Block_Attn_Mask, RowWise_Attn_Full,
                      RowWise_Attn_Sliding, RowWise_Attn_Mask)

__all__ = ['rowwise_attn_full_op', 'rowwise_attn_sliding_op', 'rowwise_attn_mask_op', 'block_attn_mask_op']
