"""Import path of the reference's mask module (``from util.masks import ...``,
src/util/masks.py:10-184)."""
from stof.masks import (generate_causal_mask, generate_sliding_mask, generate_dilated_mask,  # noqa: F401
                        generate_longformer_mask, generate_bigbird_mask, get_sparse_storage,
                        get_sparse_storage_batched, expand_sparse_storage)
