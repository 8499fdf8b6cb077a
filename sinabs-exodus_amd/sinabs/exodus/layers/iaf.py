"""Import path of the reference (sinabs/exodus/layers/iaf.py); the layers live in ``neurons``."""
from .neurons import IAF, IAFSqueeze  # noqa: F401
