"""EXODUS ``IAF`` layer (API of reference sinabs/exodus/layers/iaf.py)."""
from typing import Callable, Optional, Union

import numpy as np
import torch

from .._compat import MembraneSubtract, MultiSpike, SingleExponential, SqueezeMixin
from .lif import LIF

__all__ = ["IAF", "IAFSqueeze"]


class IAF(LIF):
    """
    Integrate-and-fire layer: a ``LIF`` whose membrane does not leak (alpha = 1) and whose input
    is not normalised.

    .. math ::
        V_{mem}(t+1) = V_{mem}(t) + \\sum z(t)

        \\text{if } V_{mem}(t) >= V_{th} \\text{, then } V_{mem} \\rightarrow V_{mem} - V_{sub}

    Parameters are those of ``LIF`` without ``tau_mem``, ``train_alphas`` and ``norm_input``.
    """

    def __init__(
        self,
        spike_threshold: Optional[Union[float, torch.Tensor]] = 1.0,
        spike_fn: Callable = MultiSpike,
        reset_fn: Callable = MembraneSubtract(),
        surrogate_grad_fn: Callable = SingleExponential(),
        tau_syn: Optional[Union[float, torch.Tensor]] = None,
        min_v_mem: Optional[Union[float, torch.Tensor]] = None,
        shape: Optional[torch.Size] = None,
        record_states: bool = False,
        decay_early: bool = True,
    ):
        super().__init__(
            tau_mem=np.inf,
            tau_syn=tau_syn,
            spike_threshold=spike_threshold,
            spike_fn=spike_fn,
            reset_fn=reset_fn,
            surrogate_grad_fn=surrogate_grad_fn,
            min_v_mem=min_v_mem,
            shape=shape,
            norm_input=False,
            record_states=record_states,
            decay_early=decay_early,
        )
        # no membrane time constant (reference iaf.py:80-81)
        self.tau_mem = None

    @property
    def alpha_mem_calculated(self):
        return torch.tensor(1.0).to(self.v_mem.device)

    @property
    def _param_dict(self) -> dict:
        param_dict = super()._param_dict
        for key in ("tau_mem", "train_alphas", "norm_input"):
            param_dict.pop(key)
        return param_dict


class IAFSqueeze(IAF, SqueezeMixin):
    """``IAF`` for squeezed 4-D input (batch*time, channel, height, width)."""

    def __init__(self, batch_size=None, num_timesteps=None, **kwargs):
        super().__init__(**kwargs)
        self.squeeze_init(batch_size, num_timesteps)

    def forward(self, input_data: torch.Tensor) -> torch.Tensor:
        return self.squeeze_forward(input_data, super().forward)

    @property
    def _param_dict(self) -> dict:
        return self.squeeze_param_dict(super()._param_dict)
