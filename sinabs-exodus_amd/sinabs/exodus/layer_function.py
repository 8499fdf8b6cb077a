"""``SpikingLayerFunction``: a whole LIF/IAF layer pass on the layer's own (batch, time, neurons)
layout, one kernel per direction.

What the reference layer does with two transposing copies, up to two autograd Functions and
several elementwise passes (reference sinabs/exodus/layers/lif.py:152-307) happens here inside
the kernels: synaptic current, input normalisation, membrane update, clamp, threshold, reset,
final states and the spike total for ``firing_rate``.  The forward keeps only checkpoints; the
backward re-reads the input and rebuilds membrane potential and synaptic current chunk by chunk,
so neither is ever written to memory in full.

A surrogate gradient the kernels do not know (any callable, as in the reference,
sinabs/exodus/spike.py:251) costs one more tensor each way: the forward also records the
potential before the reset, the backward calls the function on it and hands the result to the kernel.
"""
from typing import Callable, Optional

import torch

from . import _hip
from ._validate import check_parameters
from .spike import classify_surrogate


def _one_value(grad: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """The single element that ``grad`` repeats everywhere, as a one-element tensor -- or None when ``grad`` is an
    ordinary tensor.  The gradient of ``output.sum()`` (or of a multiple of it) arrives as a scalar expanded with
    strides of zero; the kernels take the scalar itself and read one tensor less, instead of the expansion being
    written out to memory first."""
    if grad is None or grad.numel() < 2 or any(grad.stride()) or grad.dtype != torch.float32:
        return None
    return grad.as_strided((1,), (1,))


class SpikingLayerFunction(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        inp: torch.Tensor,                      # (batch, time, neurons), contiguous
        alpha_mem: torch.Tensor,                # (batch*neurons,)
        alpha_syn: Optional[torch.Tensor],      # (batch*neurons,) or None: no synaptic current
        v_mem_init: torch.Tensor,               # (batch*neurons,) potential after reset
        i_syn_init: Optional[torch.Tensor],     # (batch*neurons,) or None
        threshold: torch.Tensor,
        membrane_subtract: Optional[torch.Tensor],
        min_v_mem: Optional[torch.Tensor],
        surrogate_grad_fn: Callable,
        max_num_spikes_per_bin: Optional[int],
        decay_early: bool,
        norm_input: bool,
        state_shape: Optional[tuple] = None,
        record_states: bool = False,
        check_values: bool = True,
    ):
        """Returns ``(spikes (batch,time,neurons), v_mem_last, i_syn_last | None, spike_total, v_mem_record |
        None, i_syn_record | None)``; ``v_mem_last`` is the potential after the last reset, ``spike_total`` a
        float64 scalar (the sum of ``spikes``; a gradient arriving at it is added to every element of the
        gradient of ``spikes``).  The final states come as flat vectors, or in ``state_shape`` if given.
        With ``record_states`` the potential after each reset and the synaptic current of every step come
        back as (batch,time,neurons) tensors, differentiable like every other output (what the layer keeps
        in ``recordings``, reference sinabs/exodus/layers/lif.py:256,290-293).  ``check_values=False`` skips
        the range checks of ``alpha`` / ``threshold`` (for a caller that knows they passed already)."""
        kind, p0, p1 = classify_surrogate(surrogate_grad_fn)
        if inp.ndim != 3:
            raise ValueError("'inp' must be 3D, (batch, time, neurons)")
        if not inp.is_contiguous():
            raise ValueError("'inp' has to be contiguous.")
        if membrane_subtract is None:
            membrane_subtract = threshold
        syn = alpha_syn is not None
        apply_min = min_v_mem is not None
        if check_values:
            check_parameters([alpha_mem, alpha_syn] if syn else [alpha_mem], threshold, min_v_mem)

        max_spikes = -1 if max_num_spikes_per_bin is None else int(max_num_spikes_per_bin)
        need_grad = any(ctx.needs_input_grad)
        res = _hip.layerLifForward(
            inp, v_mem_init, i_syn_init, alpha_mem, alpha_syn, membrane_subtract, threshold, min_v_mem, apply_min,
            max_spikes, decay_early, norm_input, wantCheckpoints=need_grad, stateShape=state_shape,
            wantPreReset=need_grad and kind == _hip.SURR_TENSOR and not record_states,
            wantRecords=bool(record_states),
        )
        ctx.cfg = (syn, apply_min, max_spikes, bool(decay_early), bool(norm_input), kind, p0, p1)
        ctx.surrogate_grad_fn = surrogate_grad_fn if kind == _hip.SURR_TENSOR else None
        ctx.set_materialize_grads(False)
        if need_grad:
            saved = [inp, res["ckpt_v"], v_mem_init, alpha_mem, membrane_subtract, threshold]
            if kind == _hip.SURR_TENSOR:
                # the function's argument is the potential before the reset; a post-reset record plus
                # what the reset took away gives it back (up to one rounding)
                v_pre = res["v_rec"]
                if record_states:
                    v_pre = torch.addcmul(v_pre, res["spikes"], membrane_subtract.view(inp.shape[0], 1, inp.shape[2]))
                saved.append(v_pre)
            if syn:
                saved += [res["ckpt_i"], i_syn_init, alpha_syn]
            if apply_min:
                saved.append(min_v_mem)
            ctx.save_for_backward(*saved)
        return (res["spikes"], res["v_last"], res["i_last"] if syn else None, res["spike_sum"],
                res["v_rec"] if record_states else None, res["i_rec"] if (record_states and syn) else None)

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_last, grad_i_last, grad_total, grad_v_rec=None, grad_i_rec=None):
        syn, apply_min, max_spikes, decay_early, norm_input, kind, p0, p1 = ctx.cfg
        saved = list(ctx.saved_tensors)
        inp, ckpt_v, v_mem_init, alpha_mem, membrane_subtract, threshold = saved[:6]
        rest = saved[6:]
        v_pre = None
        if kind == _hip.SURR_TENSOR:
            v_pre, rest = rest[0], rest[1:]
        ckpt_i = i_syn_init = alpha_syn = None
        if syn:
            ckpt_i, i_syn_init, alpha_syn = rest[:3]
            rest = rest[3:]
        min_v_mem = rest[0] if apply_min else None
        need = ctx.needs_input_grad
        if all(g is None for g in (grad_spikes, grad_v_last, grad_i_last, grad_total, grad_v_rec, grad_i_rec)):
            return (None,) * 15
        # one value for every spike (a sum as the loss, the spike total behind firing_rate): handed over as it is
        uniform = None
        if kind != _hip.SURR_TENSOR and grad_v_rec is None and grad_i_rec is None and inp.numel() > 1:
            if grad_spikes is None:
                uniform = torch.zeros(1, dtype=torch.float32, device=inp.device) if grad_total is None else None
            else:
                uniform = _one_value(grad_spikes)
            if grad_total is not None and (uniform is not None or grad_spikes is None):
                total = grad_total.to(torch.float32).reshape(1)   # d(sum of spikes) / d(spike) = 1 for every element
                uniform = total if uniform is None else uniform + total
        if uniform is not None:
            grad_spikes = uniform
        else:
            if grad_spikes is None:
                grad_spikes = torch.zeros_like(inp)
            if grad_total is not None:
                grad_spikes = grad_spikes + grad_total.to(grad_spikes.dtype)
        cont = lambda x: None if x is None else x.contiguous()
        surr = None
        if v_pre is not None:
            # the function sees (batch, time, neurons) potentials and thresholds that broadcast over time
            b, _, m = inp.shape
            with torch.no_grad():
                surr = ctx.surrogate_grad_fn(v_pre, threshold.view(b, 1, m))
            surr = torch.as_tensor(surr, device=inp.device).to(torch.float32).expand(inp.shape).contiguous()
        grad_input, g_am, g_as, g_v0, g_i0 = _hip.layerLifBackward(
            cont(grad_spikes), cont(grad_v_last), cont(grad_i_last) if syn else None, inp, ckpt_v, ckpt_i,
            v_mem_init, i_syn_init, alpha_mem, alpha_syn, membrane_subtract, threshold, min_v_mem, apply_min,
            max_spikes, decay_early, norm_input, kind, p0, p1, surr=surr,
            gradVRec=cont(grad_v_rec), gradIRec=cont(grad_i_rec) if syn else None,
            wantAlphaMemGrad=need[1], wantAlphaSynGrad=need[2], wantVInitGrad=need[3], wantIInitGrad=need[4],
            gradUniform=uniform is not None,
        )
        return (grad_input if need[0] else None, g_am, g_as, g_v0, g_i0) + (None,) * 10


class LeakyLayerFunction(torch.autograd.Function):
    """The non-spiking leaky-integrator layer (ExpLeak) on (batch, time, neurons): input scalings and
    the integrator in one kernel per direction (reference sinabs/exodus/layers/lif.py:206-223)."""

    @staticmethod
    def forward(ctx, inp, alpha, v_mem_init, decay_early: bool, norm_input: bool, state_shape=None):
        """Returns ``(out (batch,time,neurons), v_mem_last, out_total)``; ``out_total`` is the float64
        sum of ``out`` (a gradient arriving at it is added to every element of the gradient of ``out``)."""
        if inp.ndim != 3:
            raise ValueError("'inp' must be 3D, (batch, time, neurons)")
        if not inp.is_contiguous():
            raise ValueError("'inp' has to be contiguous.")
        out, v_last, total = _hip.layerLeakyForward(inp, v_mem_init, alpha, decay_early, norm_input,
                                                    stateShape=state_shape, wantSum=True)
        ctx.cfg = (bool(decay_early), bool(norm_input), alpha.requires_grad, tuple(inp.shape))
        ctx.set_materialize_grads(False)
        if alpha.requires_grad:
            need_x = decay_early or norm_input
            ctx.save_for_backward(alpha, v_mem_init, out, inp if need_x else None)
        else:
            ctx.save_for_backward(alpha)
        return out, v_last, total

    @staticmethod
    def backward(ctx, grad_out, grad_v_last, grad_total):
        decay_early, norm_input, need_alpha, shape = ctx.cfg
        if need_alpha:
            alpha, v_mem_init, out, inp = ctx.saved_tensors
        else:
            (alpha,) = ctx.saved_tensors
            v_mem_init = out = inp = None
        if grad_out is None and grad_v_last is None and grad_total is None:
            return (None,) * 6
        cont = lambda x: None if x is None else x.contiguous()
        numel = shape[0] * shape[1] * shape[2]
        if grad_out is None:
            uniform = torch.zeros(1, dtype=torch.float32, device=alpha.device) if grad_total is None else None
        else:
            uniform = _one_value(grad_out) if numel > 1 else None
        if grad_total is not None and (uniform is not None or grad_out is None) and numel > 1:
            total = grad_total.to(torch.float32).reshape(1)
            uniform = total if uniform is None else uniform + total
        if uniform is not None and numel > 1:
            grad_input, grad_alpha, grad_init = _hip.layerLeakyBackward(
                uniform, cont(grad_v_last), out, inp, v_mem_init, alpha, decay_early, norm_input, need_alpha, shape=shape)
            return grad_input, grad_alpha, grad_init, None, None, None
        if grad_out is None:
            grad_out = torch.zeros(shape, dtype=torch.float32, device=alpha.device)
        if grad_total is not None:
            grad_out = grad_out + grad_total.to(grad_out.dtype)
        grad_input, grad_alpha, grad_init = _hip.layerLeakyBackward(
            cont(grad_out), cont(grad_v_last), out, inp, v_mem_init, alpha, decay_early, norm_input, need_alpha)
        return grad_input, grad_alpha, grad_init, None, None, None
