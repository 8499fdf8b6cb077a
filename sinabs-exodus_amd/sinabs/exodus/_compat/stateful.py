"""Minimal stand-in for upstream ``sinabs.layers.LIF`` / ``StatefulLayer`` / ``SqueezeMixin``,
used as the base class of the EXODUS layers only when upstream sinabs is not installed.

It holds parameters, state buffers and constructor-argument bookkeeping; it has no forward
arithmetic of its own.  Attribute, parameter and buffer names follow what the reference relies
on at its call sites (reference sinabs/exodus/layers/lif.py:114-126, 174-177, 188, 204, 279;
layers/iaf.py:83-93; layers/exp_leak.py:64-72; conversion.py:30,54) so that ``state_dict`` keys
(``tau_mem`` / ``alpha_mem``, ``tau_syn`` / ``alpha_syn``, ``v_mem``, ``i_syn``) match upstream's.
Behaviour beyond those call sites is restated from memory of sinabs 1.2-2.0.
"""
from copy import deepcopy
from typing import Callable, Optional, Union

import torch
import torch.nn as nn

from .activation import MembraneSubtract, MultiSpike, SingleExponential


class StatefulLayer(nn.Module):
    """Module whose neuron states are buffers that persist between forward calls."""

    def __init__(self, state_names):
        super().__init__()
        for name in state_names:
            self.register_buffer(name, torch.zeros((0)))

    def zero_grad(self, set_to_none: bool = True) -> None:
        """Also cut the states loose from the graph of earlier forward calls."""
        for buf in self.buffers():
            buf.detach_()
        return super().zero_grad(set_to_none)

    def is_state_initialised(self) -> bool:
        return all(buf.shape != torch.Size([0]) for buf in self._buffers.values())

    def state_has_shape(self, shape) -> bool:
        shape = torch.Size(shape)
        return all(buf.shape == shape for buf in self._buffers.values())

    def init_state_with_shape(self, shape, randomize: bool = False) -> None:
        for name, buf in self.named_buffers():
            self.register_buffer(name, torch.zeros(shape, device=buf.device))
        self.reset_states(randomize=randomize)

    def reset_states(self, randomize: bool = False, value_ranges: Optional[dict] = None) -> None:
        if not self.is_state_initialised():
            return
        for name, buf in self._buffers.items():
            buf.detach_()
            if randomize:
                lo, hi = (value_ranges or {}).get(name, (0.0, 1.0))
                with torch.no_grad():
                    buf.uniform_(lo, hi)
            else:
                buf.zero_()

    @property
    def _param_dict(self) -> dict:
        """Constructor arguments that recreate this layer."""
        return dict()

    @property
    def arg_dict(self) -> dict:
        return self._param_dict

    @property
    def does_spike(self) -> bool:
        return getattr(self, "spike_fn", None) is not None

    def __repr__(self):
        shown = ("tau_mem", "tau_syn", "spike_threshold", "min_v_mem", "norm_input")
        plain = lambda v: v.item() if isinstance(v, torch.Tensor) and v.numel() == 1 else v
        parts = [f"{k}={plain(v)}" for k, v in self._param_dict.items() if k in shown and v is not None]
        return f"{self.__class__.__name__}({', '.join(parts)})"

    def __deepcopy__(self, memo=None):
        copy = self.__class__(**self._param_dict)
        # plain settings that subclasses keep outside their constructor-argument dict
        for key, val in self.__dict__.items():
            if not key.startswith("_") and isinstance(val, (bool, int, float, type(None))):
                copy.__dict__[key] = val
        for name, buf in self.named_buffers():
            copy.register_buffer(name, buf.detach().clone())
        for name, par in self.named_parameters():
            if par is not None:
                getattr(copy, name).data = par.data.clone()
        return copy


class LIF(StatefulLayer):
    """Parameter and state container of a leaky integrate-and-fire layer (no forward)."""

    def __init__(
        self,
        tau_mem: Union[float, torch.Tensor],
        tau_syn: Optional[Union[float, torch.Tensor]] = None,
        spike_threshold: Optional[Union[float, torch.Tensor]] = 1.0,
        spike_fn: Optional[Callable] = MultiSpike,
        reset_fn: Optional[Callable] = MembraneSubtract(),
        surrogate_grad_fn: Optional[Callable] = SingleExponential(),
        min_v_mem: Optional[Union[float, torch.Tensor]] = None,
        train_alphas: bool = False,
        shape: Optional[torch.Size] = None,
        norm_input: bool = True,
        record_states: bool = False,
    ):
        has_syn = tau_syn is not None
        super().__init__(state_names=["v_mem", "i_syn"] if has_syn else ["v_mem"])
        as_f32 = lambda v: torch.as_tensor(v, dtype=torch.float32).detach().clone()
        if train_alphas:
            self.alpha_mem = nn.Parameter(torch.exp(-1.0 / as_f32(tau_mem)))
            self.alpha_syn = nn.Parameter(torch.exp(-1.0 / as_f32(tau_syn))) if has_syn else None
        else:
            self.tau_mem = nn.Parameter(as_f32(tau_mem))
            self.tau_syn = nn.Parameter(as_f32(tau_syn)) if has_syn else None
        # fixed (non-trainable) parameters, so that they follow the module across devices
        self.spike_threshold = (nn.Parameter(as_f32(spike_threshold), requires_grad=False)
                                if spike_threshold is not None else None)
        self.spike_fn = spike_fn
        self.reset_fn = reset_fn
        self.surrogate_grad_fn = surrogate_grad_fn
        self.min_v_mem = nn.Parameter(as_f32(min_v_mem), requires_grad=False) if min_v_mem is not None else None
        self.train_alphas = train_alphas
        self.norm_input = norm_input
        self.record_states = record_states
        self.recordings = dict()
        if shape:
            self.init_state_with_shape(shape)

    @property
    def alpha_mem_calculated(self) -> torch.Tensor:
        return self.alpha_mem if self.train_alphas else torch.exp(-1.0 / self.tau_mem)

    @property
    def alpha_syn_calculated(self) -> Optional[torch.Tensor]:
        if self.train_alphas:
            return self.alpha_syn
        return None if self.tau_syn is None else torch.exp(-1.0 / self.tau_syn)

    @property
    def tau_mem_calculated(self) -> Optional[torch.Tensor]:
        if self.train_alphas:
            return -1.0 / torch.log(self.alpha_mem)
        return self.tau_mem

    @property
    def tau_syn_calculated(self) -> Optional[torch.Tensor]:
        if self.train_alphas:
            return None if self.alpha_syn is None else -1.0 / torch.log(self.alpha_syn)
        return self.tau_syn

    @property
    def _param_dict(self) -> dict:
        d = super()._param_dict
        tau_mem, tau_syn = self.tau_mem_calculated, self.tau_syn_calculated
        d.update(
            tau_mem=None if tau_mem is None else tau_mem.detach(),
            tau_syn=None if tau_syn is None else tau_syn.detach(),
            spike_threshold=self.spike_threshold,
            spike_fn=self.spike_fn,
            reset_fn=self.reset_fn,
            surrogate_grad_fn=self.surrogate_grad_fn,
            train_alphas=self.train_alphas,
            shape=self.v_mem.shape,
            min_v_mem=self.min_v_mem,
            norm_input=self.norm_input,
            record_states=self.record_states,
        )
        return d

    def forward(self, input_data):
        raise NotImplementedError("this base class only holds parameters and states")


class SqueezeMixin:
    """(batch*time, ...) <-> (batch, time, ...) reshaping for layers living between 4-D modules."""

    def squeeze_init(self, batch_size: Optional[int], num_timesteps: Optional[int]):
        if not batch_size and not num_timesteps:
            raise TypeError("You need to specify either batch_size or num_timesteps.")
        self.batch_size = batch_size if batch_size else -1
        self.num_timesteps = num_timesteps if num_timesteps else -1

    def squeeze_forward(self, input_data: torch.Tensor, forward_method: Callable):
        inflated = input_data.reshape(self.batch_size, self.num_timesteps, *input_data.shape[1:])
        return forward_method(inflated).flatten(start_dim=0, end_dim=1)

    def squeeze_param_dict(self, param_dict: dict) -> dict:
        param_dict.update(batch_size=self.batch_size, num_timesteps=self.num_timesteps)
        return param_dict


def replace_module(model: nn.Module, source_class: type, mapper_fn: Callable) -> nn.Module:
    """Copy of ``model`` in which every module whose type is exactly ``source_class`` is replaced
    by ``mapper_fn(module)``; the original model is left untouched."""
    if type(model) is source_class:
        return mapper_fn(model)
    model = deepcopy(model)
    _replace_in_place(model, source_class, mapper_fn)
    return model


def _replace_in_place(module: nn.Module, source_class: type, mapper_fn: Callable) -> None:
    for name, child in list(module.named_children()):
        if type(child) is source_class:
            setattr(module, name, mapper_fn(child))
        else:
            _replace_in_place(child, source_class, mapper_fn)
