"""TEST INFRASTRUCTURE ONLY -- CPU checker, never imported by the shipped package.

Plain (non-EXODUS) layer classes in the style of upstream ``sinabs.layers``: same constructor
arguments, parameters and state buffers as the EXODUS layers, but the forward pass is the Python
loop over time steps of ``oracle/sinabs_cpu.py`` differentiated by torch autograd.  They play the
role that ``sinabs.layers.{LIF, IAF, ExpLeak}(+Squeeze)`` play in the reference's own tests
(reference tests/test_lif.py, tests/test_iaf.py, tests/test_exp_leak.py, tests/test_conversion.py).

Restated from memory of upstream sinabs (not in the reference tree): parity with upstream is
UNPINNED; see the header of ``sinabs_cpu.py`` for what corroborates the step order.
"""
from typing import Optional

import numpy as np
import torch

from sinabs.exodus._compat import activation as act
from sinabs.exodus._compat.stateful import LIF as _Base
from sinabs.exodus._compat.stateful import SqueezeMixin

from . import sinabs_cpu as sc


def _cap(spike_fn) -> Optional[int]:
    if isinstance(spike_fn, act.MaxSpike):
        return spike_fn.max_num_spikes_per_bin
    if spike_fn is act.SingleSpike:
        return 1
    return None


class LIF(_Base):
    clip_mode = "relu"

    def forward(self, input_data: torch.Tensor) -> torch.Tensor:
        batch, steps, *trailing = input_data.shape
        if not self.is_state_initialised() or not self.state_has_shape((batch, *trailing)):
            self.init_state_with_shape((batch, *trailing))
        state = {"v_mem": self.v_mem}
        alpha_syn = self.alpha_syn_calculated
        if alpha_syn is not None:
            state["i_syn"] = self.i_syn
        spiking = self.spike_fn is not None
        sub = self.reset_fn.subtract_value if spiking else None
        out, state, rec = sc.lif_forward(
            input_data, self.alpha_mem_calculated, alpha_syn, state, self.spike_threshold, sub,
            self.surrogate_grad_fn, _cap(self.spike_fn), self.min_v_mem, self.norm_input, spiking=spiking,
            clip_mode=self.clip_mode)
        self.v_mem = state["v_mem"]
        if alpha_syn is not None:
            self.i_syn = state["i_syn"]
        self.recordings = {"v_mem": rec["v_mem_post"] if spiking else rec["v_mem"]} if self.record_states else {}
        if self.record_states and alpha_syn is not None:
            self.recordings["i_syn"] = rec["i_syn"]
        self.firing_rate = out.sum() / out.numel()
        return out


class IAF(LIF):
    def __init__(self, spike_threshold=1.0, spike_fn=act.MultiSpike, reset_fn=act.MembraneSubtract(),
                 surrogate_grad_fn=act.SingleExponential(), tau_syn=None, min_v_mem=None, shape=None,
                 record_states=False):
        super().__init__(tau_mem=np.inf, tau_syn=tau_syn, spike_threshold=spike_threshold, spike_fn=spike_fn,
                         reset_fn=reset_fn, surrogate_grad_fn=surrogate_grad_fn, min_v_mem=min_v_mem, shape=shape,
                         norm_input=False, record_states=record_states)
        self.tau_mem = None

    @property
    def alpha_mem_calculated(self):
        return torch.tensor(1.0).to(self.v_mem.device)

    @property
    def _param_dict(self) -> dict:
        d = super()._param_dict
        for k in ("tau_mem", "train_alphas", "norm_input"):
            d.pop(k)
        return d


class ExpLeak(LIF):
    def __init__(self, tau_mem, shape=None, train_alphas=False, min_v_mem=None, norm_input=False,
                 record_states=False):
        super().__init__(tau_mem=tau_mem, tau_syn=None, spike_threshold=None, train_alphas=train_alphas,
                         min_v_mem=min_v_mem, shape=shape, spike_fn=None, reset_fn=None, surrogate_grad_fn=None,
                         norm_input=norm_input, record_states=record_states)

    @property
    def _param_dict(self) -> dict:
        d = super()._param_dict
        for k in ("tau_syn", "spike_fn", "reset_fn", "surrogate_grad_fn", "spike_threshold"):
            d.pop(k)
        return d


def _squeeze(cls):
    class Squeezed(cls, SqueezeMixin):
        def __init__(self, batch_size=None, num_timesteps=None, **kwargs):
            super().__init__(**kwargs)
            self.squeeze_init(batch_size, num_timesteps)

        def forward(self, input_data):
            return self.squeeze_forward(input_data, super().forward)

        @property
        def _param_dict(self) -> dict:
            return self.squeeze_param_dict(super()._param_dict)

    Squeezed.__name__ = Squeezed.__qualname__ = cls.__name__ + "Squeeze"
    return Squeezed


LIFSqueeze = _squeeze(LIF)
IAFSqueeze = _squeeze(IAF)
ExpLeakSqueeze = _squeeze(ExpLeak)
