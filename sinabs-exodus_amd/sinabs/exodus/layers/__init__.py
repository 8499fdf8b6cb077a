"""``sinabs.exodus.layers``: LIF, IAF, ExpLeak and their Squeeze variants."""
from .neurons import ExpLeak, ExpLeakSqueeze, IAF, IAFSqueeze, LIF, LIFSqueeze  # noqa: F401

__all__ = ["LIF", "LIFSqueeze", "IAF", "IAFSqueeze", "ExpLeak", "ExpLeakSqueeze"]
