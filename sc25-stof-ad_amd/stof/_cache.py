"""What the per-tensor caches of the operators are keyed on, shared by the LUT compiler (which
can hand over bit rows it has already built) and the attention operators (which use them)."""

BITS_ATTR = "_stof_packed_bits"       # on part_block_mask / row_mask: (content key, packed bit rows)
LUT_OK_ATTR = "_stof_lut_checked"     # on load_col_idx: content keys of the four index tensors found in order
DEVICE_BUILT_ATTR = "_stof_device_built"   # on tensors the library's kernels produced: their attached data is not re-derivable


def content_key(t):
    """The storage address and PyTorch's in-place version counter.  A write that goes around
    PyTorch (another library through ``data_ptr``, DLPack, numpy-shared memory) changes neither:
    such callers pass ``revalidate=True`` to the operator."""
    return (t.data_ptr(), t._version)
