"""Import path of the reference (sinabs/exodus/layers/exp_leak.py); the layers live in ``neurons``."""
from .neurons import ExpLeak, ExpLeakSqueeze  # noqa: F401
