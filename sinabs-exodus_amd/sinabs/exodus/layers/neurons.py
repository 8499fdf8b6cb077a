"""The EXODUS neuron layers on the gfx950 kernels: ``LIF`` and its two specialisations ``IAF`` (no leak,
no input normalisation) and ``ExpLeak`` (no spikes), plus the ``*Squeeze`` variants for 4-D
(batch*time, channel, height, width) tensors.

Public names, constructor arguments, parameters, states and outputs are those of the reference
layers (reference sinabs/exodus/layers/lif.py, iaf.py, exp_leak.py); the modules ``lif``, ``iaf`` and
``exp_leak`` next to this one re-export them under the reference's import paths.
"""
from typing import Callable, Optional, Tuple, Union

import numpy as np
import torch

from .._compat import (LIFBase, MaxSpike, MembraneSubtract, MultiSpike, SingleExponential, SingleSpike,
                       SqueezeMixin)
from .. import _hip
from .._validate import check_parameters
from ..leaky import LeakyIntegrator
from ..layer_function import LeakyLayerFunction, SpikingLayerFunction
from ..spike import IntegrateAndFire
from ..synaptic import SynapticIntegrateAndFire, fusable

__all__ = ["LIF", "LIFSqueeze", "IAF", "IAFSqueeze", "ExpLeak", "ExpLeakSqueeze", "expand_to_1d_contiguous"]


def expand_to_1d_contiguous(value: Union[float, torch.Tensor], shape: Tuple[int], device=None) -> torch.Tensor:
    """Broadcast ``value`` to ``shape`` (so per-channel tensors line up with the batch dimension),
    then flatten to a contiguous float32 vector with one entry per row of the (N, T) matrices
    (reference sinabs/exodus/layers/lif.py:20-44).  ``device`` moves plain numbers and stray CPU
    tensors next to the states; a plain number is written by a fill kernel rather than copied from
    host memory, which also works while a HIP graph is being captured."""
    if not isinstance(value, torch.Tensor):
        return torch.full((int(np.prod(shape)),), float(value), dtype=torch.float32, device=device)
    return torch.as_tensor(value, device=device).expand(shape).float().flatten().contiguous()


class LIF(LIFBase):
    """
    Leaky integrate-and-fire layer whose dynamics and gradients run in HIP kernels.

    Neuron dynamics in discrete time:

    .. math ::
        V_{mem}(t+1) = \\alpha V_{mem}(t) + (1-\\alpha)\\sum z(t)

        \\text{if } V_{mem}(t) >= V_{th} \\text{, then } V_{mem} \\rightarrow V_{mem} - V_{sub}

    with :math:`\\alpha = e^{-1/\\tau_{mem}}`.

    Parameters
    ----------
    tau_mem: membrane time constant.
    tau_syn: synaptic time constant; None (default) means no synaptic dynamics.
    spike_threshold: spikes are emitted when v_mem reaches this value. Default 1.0.
    spike_fn: ``MultiSpike`` / ``SingleSpike`` (pass the class) or a ``MaxSpike(k)`` instance.
    reset_fn: a ``MembraneSubtract`` instance (the only supported reset).
    surrogate_grad_fn: callable ``(v_mem, threshold) -> d spikes / d v_mem``.
    min_v_mem: lower bound of v_mem, applied at every step; None = unbounded.
    train_alphas: train the decay factors exp(-1/tau) instead of the time constants.
    shape: optionally initialise the state with this shape; otherwise inferred from the input.
    norm_input: scale the input current by (1 - alpha_mem).
    record_states: keep v_mem / i_syn of every step in ``self.recordings``.
    decay_early: apply the synaptic decay to an input already in the step it arrives, so that a
        unit pulse gives a synaptic current of alpha rather than one (same as sinabs). Only
        affects synaptic currents. Default True.
    """

    def __init__(
        self,
        tau_mem: Union[float, torch.Tensor],
        tau_syn: Optional[Union[float, torch.Tensor]] = None,
        spike_threshold: Optional[Union[float, torch.Tensor]] = 1.0,
        spike_fn: Callable = MultiSpike,
        reset_fn: Callable = MembraneSubtract(),
        surrogate_grad_fn: Callable = SingleExponential(),
        min_v_mem: Optional[Union[float, torch.Tensor]] = None,
        train_alphas: bool = False,
        shape: Optional[torch.Size] = None,
        norm_input: bool = True,
        record_states: bool = False,
        decay_early: bool = True,
    ):
        self._parse_activation_fn(spike_fn, reset_fn)
        super().__init__(
            tau_mem=tau_mem,
            tau_syn=tau_syn,
            spike_threshold=spike_threshold,
            spike_fn=spike_fn,
            reset_fn=reset_fn,
            surrogate_grad_fn=surrogate_grad_fn,
            min_v_mem=min_v_mem,
            train_alphas=train_alphas,
            shape=shape,
            norm_input=norm_input,
            record_states=record_states,
        )
        self.decay_early = decay_early
        # layers with synapses run synapse and membrane in one kernel when the surrogate gradient
        # is one the kernels can evaluate; set to False to force the two separate Functions
        self.fuse_synapse = True
        # float32 device inputs run one kernel per direction on the input's own (batch, time, neurons)
        # layout (no transposing copies, no stored v_mem / i_syn); set to False to force the
        # (rows, time) Functions
        self.native_layout = True

    def _parse_activation_fn(self, spike_fn, reset_fn):
        """Translate the spike mechanism into a per-step spike cap (reference lif.py:130-150)."""
        if spike_fn is None:
            return  # non-spiking
        supported_spike = spike_fn in (MultiSpike, SingleSpike) or isinstance(spike_fn, MaxSpike)
        if not supported_spike or not isinstance(reset_fn, MembraneSubtract):
            raise NotImplementedError(
                "Spike mechanism config not supported. "
                "Use MultiSpike/SingleSpike/MaxSpike and MembraneSubtract functions."
            )
        if isinstance(spike_fn, MaxSpike):
            self.max_num_spikes_per_bin = spike_fn.max_num_spikes_per_bin
        elif spike_fn == MultiSpike:
            self.max_num_spikes_per_bin = None
        else:
            self.max_num_spikes_per_bin = 1

    # ------------------------------------------------------------------ layout
    def _prepare_input(self, input_data: torch.Tensor):
        """(batch, time, *trailing) -> contiguous (batch*prod(trailing), time); (re)initialise the
        states when their shape does not fit (reference lif.py:152-183)."""
        batch_size, time_steps, *trailing_dim = input_data.shape
        state_shape = (batch_size, *trailing_dim)
        if not self.is_state_initialised() or not self.state_has_shape(state_shape):
            self.init_state_with_shape(state_shape)
        input_2d = input_data.movedim(1, -1).reshape(-1, time_steps)
        return input_2d, (batch_size, time_steps, *trailing_dim)

    @staticmethod
    def _rows_to_full(x_2d: torch.Tensor, batch_size: int, trailing_dim) -> torch.Tensor:
        return x_2d.reshape(batch_size, *trailing_dim, -1).movedim(-1, 1)

    # ------------------------------------------------------------------ dynamics
    def _forward_synaptic(self, input_2d: torch.Tensor) -> torch.Tensor:
        """Exponential synapse i_t = alpha_syn * i_{t-1} + x_t (x pre-scaled by alpha_syn when
        ``decay_early``) -- reference lif.py:185-198."""
        alpha_syn = expand_to_1d_contiguous(self.alpha_syn_calculated, self.v_mem.shape, self.v_mem.device)
        if self.decay_early:
            input_2d = input_2d * alpha_syn.unsqueeze(1)
        return LeakyIntegrator.apply(input_2d.contiguous(), alpha_syn, self.i_syn.flatten().contiguous())

    def _forward_membrane(self, i_syn_2d: torch.Tensor):
        """Membrane stage: returns (output, post-reset v_mem), both (N, T) -- reference lif.py:200-258."""
        state_shape = self.v_mem.shape
        dev = self.v_mem.device
        alpha_mem = expand_to_1d_contiguous(self.alpha_mem_calculated, state_shape, dev)

        if self.norm_input:
            i_syn_2d = (1.0 - alpha_mem.unsqueeze(1)) * i_syn_2d

        if self.spike_fn is None:
            # leaky integrator without spikes: output and state are the same tensor
            if self.decay_early:
                i_syn_2d = i_syn_2d * alpha_mem.unsqueeze(1)
            v_mem = LeakyIntegrator.apply(i_syn_2d.contiguous(), alpha_mem, self.v_mem.flatten().contiguous())
            return v_mem, v_mem

        spike_threshold = expand_to_1d_contiguous(self.spike_threshold, state_shape, dev)
        min_v_mem = None if self.min_v_mem is None else expand_to_1d_contiguous(self.min_v_mem, state_shape, dev)
        membrane_subtract = self.reset_fn.subtract_value
        if membrane_subtract is None:
            membrane_subtract = spike_threshold
        else:
            membrane_subtract = expand_to_1d_contiguous(membrane_subtract, state_shape, dev)

        output_2d, v_mem_2d = IntegrateAndFire.apply(
            i_syn_2d.contiguous(),
            alpha_mem,
            self.v_mem.flatten().contiguous(),
            spike_threshold,
            membrane_subtract,
            min_v_mem,
            self.surrogate_grad_fn,
            self.max_num_spikes_per_bin,
        )
        # the Function returns the potential before reset; the layer state is after reset
        v_mem_2d = v_mem_2d - membrane_subtract.unsqueeze(1) * output_2d
        return output_2d, v_mem_2d

    def _forward_synaptic_membrane(self, input_2d: torch.Tensor):
        """Same values as ``_forward_synaptic`` followed by ``_forward_membrane`` (same operations
        in the same order), computed by the fused kernels: returns (output, post-reset v_mem, i_syn)."""
        state_shape, dev = self.v_mem.shape, self.v_mem.device
        alpha_syn = expand_to_1d_contiguous(self.alpha_syn_calculated, state_shape, dev)
        alpha_mem = expand_to_1d_contiguous(self.alpha_mem_calculated, state_shape, dev)
        spike_threshold = expand_to_1d_contiguous(self.spike_threshold, state_shape, dev)
        min_v_mem = None if self.min_v_mem is None else expand_to_1d_contiguous(self.min_v_mem, state_shape, dev)
        membrane_subtract = self.reset_fn.subtract_value
        if membrane_subtract is None:
            membrane_subtract = spike_threshold
        else:
            membrane_subtract = expand_to_1d_contiguous(membrane_subtract, state_shape, dev)
        output_2d, v_mem_2d, i_syn_2d = SynapticIntegrateAndFire.apply(
            input_2d.contiguous(),
            alpha_syn,
            alpha_mem,
            self.i_syn.flatten().contiguous(),
            self.v_mem.flatten().contiguous(),
            spike_threshold,
            membrane_subtract,
            min_v_mem,
            self.surrogate_grad_fn,
            self.max_num_spikes_per_bin,
            self.decay_early,
            self.norm_input,
        )
        v_mem_2d = v_mem_2d - membrane_subtract.unsqueeze(1) * output_2d
        return output_2d, v_mem_2d, i_syn_2d

    def _use_native_layout(self, input_data: torch.Tensor) -> bool:
        if not (self.native_layout and input_data.is_cuda and input_data.dtype == torch.float32
                and input_data.ndim >= 2):
            return False
        if int(np.prod(input_data.shape[2:])) >= _hip.LAYER_MAX_NEURONS:   # the kernels keep step offsets in 32 bits
            return False
        if self.spike_fn is None:                      # leaky integrator: the output is the state record
            return self.tau_syn_calculated is None
        return True

    def _decay_source(self, which: str):
        """The parameter a decay factor derives from: the factor itself or its time constant (None for a
        layer without leak, whose factor is the constant 1)."""
        return getattr(self, ("alpha_" if self.train_alphas else "tau_") + which, None)

    def _value_stamp(self, state_shape):
        """Identity and version of everything the range checks depend on.  The checks of decay factors,
        threshold and lower bound make the host wait for the device (reference sinabs/exodus/spike.py:183-191
        does so on every call).  The layer's own parameters only change between calls when somebody writes
        to them, which their version counters show, so a layer whose parameters passed once skips the
        checks until one of them is modified, replaced or moved (a write through ``tensor.data`` bypasses
        the counter and is only seen together with the next ordinary write)."""
        def stamp(name):
            v = getattr(self, name, None)
            if isinstance(v, torch.Tensor):
                return (id(v), v._version, v.data_ptr(), tuple(v.shape))
            return v
        names = ("tau_mem", "alpha_mem", "tau_syn", "alpha_syn", "spike_threshold", "min_v_mem")
        return tuple(stamp(n) for n in names) + (tuple(state_shape),)

    def _per_neuron(self, name: str, source, state_shape, dev, value=None) -> torch.Tensor:
        """One float32 entry per neuron of ``state_shape`` for the layer quantity ``name``
        (``expand_to_1d_contiguous``).  ``source`` is the parameter or number it derives from and ``value`` a
        callable giving the quantity itself when it is not the source (a decay factor computed from a time
        constant).  Quantities that take no part in differentiation are kept until their source is written
        to, replaced or moved: a layer call then launches no kernels for them."""
        compute = (lambda: source) if value is None else value
        if isinstance(source, torch.Tensor):
            if (source.requires_grad and torch.is_grad_enabled()) or torch.cuda.is_current_stream_capturing():
                return expand_to_1d_contiguous(compute(), state_shape, dev)
            key = (id(source), source._version, source.data_ptr(), tuple(source.shape), tuple(state_shape), str(dev))
        else:
            if torch.cuda.is_current_stream_capturing():
                return expand_to_1d_contiguous(compute(), state_shape, dev)
            key = (source, tuple(state_shape), str(dev))
        cache = self.__dict__.setdefault("_per_neuron_cache", {})
        hit = cache.get(name)
        if hit is not None and hit[0] == key:
            return hit[1]
        out = expand_to_1d_contiguous(compute(), state_shape, dev).detach()
        cache[name] = (key, out)
        return out

    def _set_state(self, name: str, value: torch.Tensor) -> None:
        """Replace a state buffer (``nn.Module.__setattr__`` does the same after a longer search)."""
        if name in self._buffers:
            self._buffers[name] = value
        else:
            setattr(self, name, value)

    def _needs_grad(self, input_data: torch.Tensor) -> bool:
        if not torch.is_grad_enabled():
            return False
        return (input_data.requires_grad or any(p is not None and p.requires_grad for p in self._parameters.values())
                or any(b is not None and b.requires_grad for b in self._buffers.values()))

    # ``firing_rate`` (spikes per neuron and step of the last call, reference lif.py:305) is worked out when somebody
    # asks for it: the kernels hand back the spike total, and dividing it costs two more kernel launches that a
    # training loop which never looks at the rate need not pay.  It stays differentiable (the total is an output of the
    # autograd Function).  Assigning to the attribute works as before.
    @property
    def firing_rate(self):
        parts = self.__dict__.get("_firing_rate_parts")
        if parts is not None:
            total, count = parts
            self.__dict__["_firing_rate_value"] = (total / max(count, 1)).float()
            self.__dict__["_firing_rate_parts"] = None
        return self.__dict__.get("_firing_rate_value")

    @firing_rate.setter
    def firing_rate(self, value):
        self.__dict__["_firing_rate_value"] = value
        self.__dict__["_firing_rate_parts"] = None

    def _firing_rate_from(self, total: torch.Tensor, count: int) -> None:
        self.__dict__["_firing_rate_parts"] = (total, count)

    def _forward_native_leaky(self, input_data: torch.Tensor) -> torch.Tensor:
        batch_size, time_steps, *trailing_dim = input_data.shape
        state_shape = (batch_size, *trailing_dim)
        if not self.is_state_initialised() or not self.state_has_shape(state_shape):
            self.init_state_with_shape(state_shape)
        alpha_mem = self._per_neuron("alpha_mem", self._decay_source("mem"), state_shape, self.v_mem.device,
                                     lambda: self.alpha_mem_calculated)
        out, v_last, total = LeakyLayerFunction.apply(
            input_data.reshape(batch_size, time_steps, int(np.prod(trailing_dim))).contiguous(),
            alpha_mem,
            self.v_mem.flatten().contiguous(),
            self.decay_early,
            self.norm_input,
            state_shape,
        )
        out = out.reshape(input_data.shape)
        self.recordings = {"v_mem": out} if self.record_states else dict()
        self._set_state("v_mem", v_last)
        self._firing_rate_from(total, out.numel())
        return out

    def _forward_native(self, input_data: torch.Tensor) -> torch.Tensor:
        """Whole layer in one kernel on (batch, time, neurons); same values as the other path."""
        batch_size, time_steps, *trailing_dim = input_data.shape
        state_shape = (batch_size, *trailing_dim)
        if not self.is_state_initialised() or not self.state_has_shape(state_shape):
            self.init_state_with_shape(state_shape)
        dev = self.v_mem.device
        has_syn = self.tau_syn_calculated is not None
        alpha_mem = self._per_neuron("alpha_mem", self._decay_source("mem"), state_shape, dev,
                                     lambda: self.alpha_mem_calculated)
        alpha_syn = self._per_neuron("alpha_syn", self._decay_source("syn"), state_shape, dev,
                                     lambda: self.alpha_syn_calculated) if has_syn else None
        spike_threshold = self._per_neuron("spike_threshold", self.spike_threshold, state_shape, dev)
        min_v_mem = None if self.min_v_mem is None else self._per_neuron("min_v_mem", self.min_v_mem, state_shape, dev)
        membrane_subtract = self.reset_fn.subtract_value
        if membrane_subtract is None:
            membrane_subtract = spike_threshold
        else:
            membrane_subtract = self._per_neuron("membrane_subtract", membrane_subtract, state_shape, dev)
        flat_input = input_data.reshape(batch_size, time_steps, int(np.prod(trailing_dim))).contiguous()
        stamp = self._value_stamp(state_shape)
        check_values = getattr(self, "_checked_values", None) != stamp
        if not self._needs_grad(input_data):
            # nothing to differentiate: no checkpoints, and the per-step states can be written along the way
            with torch.no_grad():
                if check_values:
                    check_parameters([alpha_mem, alpha_syn] if has_syn else [alpha_mem], spike_threshold, min_v_mem)
                    if not torch.cuda.is_current_stream_capturing():
                        self._checked_values = stamp
                res = _hip.layerLifForward(
                    flat_input, self.v_mem.flatten().contiguous(),
                    self.i_syn.flatten().contiguous() if has_syn else None, alpha_mem, alpha_syn, membrane_subtract,
                    spike_threshold, min_v_mem, min_v_mem is not None,
                    -1 if self.max_num_spikes_per_bin is None else int(self.max_num_spikes_per_bin),
                    self.decay_early, self.norm_input, wantCheckpoints=False, wantRecords=self.record_states,
                    stateShape=state_shape)
            self.recordings = dict()
            if self.record_states:
                self.recordings["v_mem"] = res["v_rec"].reshape(input_data.shape)
                if has_syn:
                    self.recordings["i_syn"] = res["i_rec"].reshape(input_data.shape)
            self._set_state("v_mem", res["v_last"])
            if has_syn:
                self._set_state("i_syn", res["i_last"])
            self._firing_rate_from(res["spike_sum"], flat_input.numel())
            return res["spikes"].reshape(input_data.shape)
        spikes, v_last, i_last, spike_total, v_rec, i_rec = SpikingLayerFunction.apply(
            flat_input,
            alpha_mem,
            alpha_syn,
            self.v_mem.flatten().contiguous(),
            self.i_syn.flatten().contiguous() if has_syn else None,
            spike_threshold,
            membrane_subtract,
            min_v_mem,
            self.surrogate_grad_fn,
            self.max_num_spikes_per_bin,
            self.decay_early,
            self.norm_input,
            state_shape,
            self.record_states,
            check_values,
        )
        if check_values and not torch.cuda.is_current_stream_capturing():
            self._checked_values = stamp
        self.recordings = dict()
        if self.record_states:
            self.recordings["v_mem"] = v_rec.reshape(input_data.shape)
            if has_syn:
                self.recordings["i_syn"] = i_rec.reshape(input_data.shape)
        self._set_state("v_mem", v_last)
        if has_syn:
            self._set_state("i_syn", i_last)
        self._firing_rate_from(spike_total, spikes.numel())
        return spikes.reshape(input_data.shape)

    def forward(self, input_data: torch.Tensor) -> torch.Tensor:
        """Process ``input_data`` of shape (batch, time, ...); returns a tensor of the same shape."""
        if self._use_native_layout(input_data):
            if self.spike_fn is None:
                return self._forward_native_leaky(input_data)
            return self._forward_native(input_data)
        input_2d, (batch_size, time_steps, *trailing_dim) = self._prepare_input(input_data)
        self.recordings = dict()

        if self.tau_syn_calculated is None:
            output_2d, v_mem_2d = self._forward_membrane(input_2d)
        else:
            if self.spike_fn is not None and self.fuse_synapse and fusable(self.surrogate_grad_fn):
                # synapse and membrane in one kernel per direction
                output_2d, v_mem_2d, i_syn_2d = self._forward_synaptic_membrane(input_2d)
            else:
                i_syn_2d = self._forward_synaptic(input_2d)
                output_2d, v_mem_2d = self._forward_membrane(i_syn_2d)
            i_syn_full = self._rows_to_full(i_syn_2d, batch_size, trailing_dim)
            self.i_syn = i_syn_full[:, -1].clone()
            if self.record_states:
                self.recordings["i_syn"] = i_syn_full

        v_mem_full = self._rows_to_full(v_mem_2d, batch_size, trailing_dim)
        output_full = self._rows_to_full(output_2d, batch_size, trailing_dim)

        if self.record_states:
            self.recordings["v_mem"] = v_mem_full
        self.v_mem = v_mem_full[:, -1].clone()
        self.firing_rate = output_full.sum() / output_full.numel()
        return output_full

    def __repr__(self):
        return "EXODUS " + super().__repr__()


class IAF(LIF):
    """
    Integrate-and-fire layer: a ``LIF`` whose membrane does not leak (alpha = 1) and whose input is
    not normalised.

    .. math ::
        V_{mem}(t+1) = V_{mem}(t) + \\sum z(t)

        \\text{if } V_{mem}(t) >= V_{th} \\text{, then } V_{mem} \\rightarrow V_{mem} - V_{sub}

    Takes the arguments of ``LIF`` except ``tau_mem``, ``train_alphas`` and ``norm_input``.
    """

    _dropped_args = ("tau_mem", "train_alphas", "norm_input")

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
        LIF.__init__(self, np.inf, tau_syn, spike_threshold, spike_fn, reset_fn, surrogate_grad_fn, min_v_mem,
                     train_alphas=False, shape=shape, norm_input=False, record_states=record_states,
                     decay_early=decay_early)
        self.tau_mem = None                      # an IAF neuron has no membrane time constant

    @property
    def alpha_mem_calculated(self):
        return torch.ones((), device=self.v_mem.device)

    @property
    def _param_dict(self) -> dict:
        return {k: v for k, v in super()._param_dict.items() if k not in self._dropped_args}


class ExpLeak(LIF):
    """
    Leaky integrator without spikes: the output is the membrane potential.

    .. math ::
        V_{mem}(t+1) = \\alpha V_{mem}(t) + (1-\\alpha)\\sum z(t)

    ``tau_mem``, ``shape``, ``train_alphas``, ``min_v_mem``, ``norm_input`` (default False here) and
    ``record_states`` as for ``LIF``.  ``decay_early`` applies the decay to an input already in the step
    it arrives, so that a unit pulse gives alpha rather than one; False (default) is the sinabs behaviour.
    """

    _dropped_args = ("tau_syn", "spike_fn", "reset_fn", "surrogate_grad_fn", "spike_threshold")

    def __init__(
        self,
        tau_mem: Union[float, torch.Tensor],
        shape: Optional[torch.Size] = None,
        train_alphas: bool = False,
        min_v_mem: Optional[float] = None,
        norm_input: bool = False,
        record_states: bool = False,
        decay_early: bool = False,
    ):
        LIF.__init__(self, tau_mem, None, None, None, None, None, min_v_mem, train_alphas, shape, norm_input,
                     record_states, decay_early)

    @property
    def _param_dict(self) -> dict:
        return {k: v for k, v in super()._param_dict.items() if k not in self._dropped_args}


def _squeezed(layer_cls: type, name: str) -> type:
    """The variant of ``layer_cls`` for squeezed 4-D input (batch*time, channel, height, width), as
    produced and consumed by convolution and pooling layers: it inflates the input to
    (batch, time, ...), runs ``layer_cls`` and flattens the first two dimensions again."""

    class Squeezed(layer_cls, SqueezeMixin):
        def __init__(self, batch_size=None, num_timesteps=None, **kwargs):
            layer_cls.__init__(self, **kwargs)
            self.squeeze_init(batch_size, num_timesteps)

        def forward(self, input_data: torch.Tensor) -> torch.Tensor:
            return self.squeeze_forward(input_data, super().forward)

        @property
        def _param_dict(self) -> dict:
            return self.squeeze_param_dict(super()._param_dict)

    Squeezed.__name__ = Squeezed.__qualname__ = name
    Squeezed.__module__ = __name__
    Squeezed.__doc__ = f"``{layer_cls.__name__}`` for squeezed 4-D input (batch*time, channel, height, width)."
    return Squeezed


LIFSqueeze = _squeezed(LIF, "LIFSqueeze")
IAFSqueeze = _squeezed(IAF, "IAFSqueeze")
ExpLeakSqueeze = _squeezed(ExpLeak, "ExpLeakSqueeze")
