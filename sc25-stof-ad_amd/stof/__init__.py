"""STOF hot path on MI355X (gfx950): block-masked multi-head attention driven by a
full / partial / empty block LUT, and fused encoder operators, behind the reference's
Python operator API.  Host code is PyTorch-ROCm; all device work is in libstof_hip.so."""
from . import masks  # noqa: F401
from ._lib import StofError, LIB_PATH  # noqa: F401
