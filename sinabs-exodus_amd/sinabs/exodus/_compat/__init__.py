"""Resolves the upstream ``sinabs`` names the EXODUS layers build on.

When upstream sinabs is importable its classes are used (the EXODUS layers then subclass the
real ``sinabs.layers.LIF``, as in the reference, sinabs/exodus/layers/lif.py:4-12).  Otherwise
the minimal stand-ins of this package are used, so that the layers can still be constructed,
run and checkpointed on a machine that only has PyTorch-ROCm.
"""
try:  # pragma: no cover - depends on the environment
    from sinabs.activation import (Heaviside, MaxSpike, MembraneSubtract, MultiSpike, PeriodicExponential,
                                   SingleExponential, SingleSpike)
    from sinabs.conversion import replace_module
    from sinabs.layers import LIF as LIFBase
    from sinabs.layers import SqueezeMixin

    HAVE_UPSTREAM_SINABS = True
except ImportError:
    from .activation import (Heaviside, MaxSpike, MembraneSubtract, MultiSpike, PeriodicExponential,
                             SingleExponential, SingleSpike)
    from .stateful import LIF as LIFBase
    from .stateful import SqueezeMixin, replace_module

    HAVE_UPSTREAM_SINABS = False

__all__ = ["Heaviside", "MaxSpike", "MembraneSubtract", "MultiSpike", "PeriodicExponential", "SingleExponential",
           "SingleSpike", "LIFBase", "SqueezeMixin", "replace_module", "HAVE_UPSTREAM_SINABS"]
