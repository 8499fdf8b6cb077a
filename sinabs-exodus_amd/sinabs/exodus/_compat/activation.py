"""Stand-ins for the parts of upstream ``sinabs.activation`` that the EXODUS layers take as
arguments, used only when upstream sinabs is not installed.

The spike and reset mechanisms are configuration markers here: the layers read which one was
chosen (reference sinabs/exodus/layers/lif.py:130-150, 237-243) and the HIP kernels do the
arithmetic.  The surrogate-gradient classes are real callables ``(v_mem, threshold) -> tensor``
made of torch operations that run on whatever device their arguments live on; the kernels
recognise these three classes and evaluate the same formulas in registers.

Formulas and default values are restated from memory of sinabs 1.2-2.0 (its source is not part
of the EXODUS repository); only ``Heaviside`` is corroborated by the reference
(Gradient_analysis.ipynb, cell 1).
"""
from dataclasses import dataclass
from typing import Optional

import torch


class MultiSpike:
    """As many spikes per step as ``v_mem`` holds multiples of the threshold. Pass the class itself."""

    required_states = ["v_mem"]


class SingleSpike:
    """At most one spike per step. Pass the class itself."""

    required_states = ["v_mem"]


@dataclass
class MaxSpike:
    """At most ``max_num_spikes_per_bin`` spikes per step. Pass an instance."""

    max_num_spikes_per_bin: Optional[int] = None
    required_states = ["v_mem"]


@dataclass
class MembraneSubtract:
    """Subtract ``subtract_value`` (default: the threshold) from ``v_mem`` for each spike."""

    subtract_value: Optional[float] = None


@dataclass
class MembraneReset:
    """Reset ``v_mem`` to a fixed value after a spike. Not supported by the EXODUS layers
    (reference sinabs/exodus/layers/lif.py:136-143 raises for anything but MembraneSubtract)."""

    reset_value: float = 0.0


@dataclass
class Heaviside:
    """1/threshold where ``v_mem >= threshold - window``, else 0."""

    window: float = 1.0

    def __call__(self, v_mem, threshold):
        return (v_mem >= (threshold - self.window)).float() / threshold


@dataclass
class SingleExponential:
    """``grad_scale / (threshold*grad_width) * exp(-|v_mem - threshold| / (threshold*grad_width))``."""

    grad_width: float = 0.5
    grad_scale: float = 1.0

    def __call__(self, v_mem, threshold):
        abs_width = threshold * self.grad_width
        return self.grad_scale / abs_width * torch.exp(-torch.abs(v_mem - threshold) / abs_width)


@dataclass
class PeriodicExponential:
    """Exponential bump around the threshold, repeated with period ``threshold`` above it."""

    grad_width: float = 0.5
    grad_scale: float = 1.0

    def __call__(self, v_mem, threshold):
        shifted = v_mem - threshold / 2
        periodic = shifted % threshold
        below = shifted * (v_mem < threshold)
        above = periodic * (v_mem >= threshold)
        folded = above + below
        pdf = torch.exp(-torch.abs(folded - threshold / 2) / self.grad_width) / threshold
        return self.grad_scale * pdf
