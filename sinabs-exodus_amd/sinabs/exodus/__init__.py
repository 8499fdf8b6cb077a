"""EXODUS spiking-neuron layers for AMD MI355X (gfx950): HIP kernels behind the
``sinabs.exodus`` API."""
__version__ = "0.1.0"

from . import conversion, layers  # noqa: F401
