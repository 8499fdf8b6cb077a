"""Import path of the reference (sinabs/exodus/layers/lif.py); the layers live in ``neurons``."""
from .neurons import LIF, LIFSqueeze, expand_to_1d_contiguous  # noqa: F401
