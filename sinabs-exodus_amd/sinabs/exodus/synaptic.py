"""``SynapticIntegrateAndFire``: synaptic current and spiking membrane in one kernel per direction.

The reference computes this stage as ``input * alpha_syn`` -> ``LeakyIntegrator`` ->
``(1 - alpha_mem) * i_syn`` -> ``IntegrateAndFire`` (reference sinabs/exodus/layers/lif.py:185-254)
with torch autograd chaining the pieces.  This Function produces the same three tensors
(spikes, pre-reset v_mem, i_syn) with the same operations in the same order, and its backward
returns what autograd would assemble from the pieces: gradients for the input, both decay
factors and both initial states.  It needs a surrogate gradient the kernels know
(``SingleExponential``, ``PeriodicExponential``, ``Heaviside``); the layer falls back to the
composed Functions for any other callable.
"""
from typing import Callable, Optional

import torch

from . import _hip
from ._checks import check_per_row, check_rows_by_time
from ._validate import check_parameters
from .spike import classify_surrogate


def fusable(surrogate_grad_fn) -> bool:
    return classify_surrogate(surrogate_grad_fn)[0] != _hip.SURR_TENSOR


class SynapticIntegrateAndFire(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        inp: torch.Tensor,
        alpha_syn: torch.Tensor,
        alpha_mem: torch.Tensor,
        i_syn_init: torch.Tensor,
        v_mem_init: torch.Tensor,
        threshold: torch.Tensor,
        membrane_subtract: Optional[torch.Tensor],
        min_v_mem: Optional[torch.Tensor],
        surrogate_grad_fn: Callable,
        max_num_spikes_per_bin: Optional[int] = None,
        decay_early: bool = True,
        norm_input: bool = True,
    ):
        """All tensors are (N, T) or (N,) as for ``IntegrateAndFire``; returns
        ``(output_spikes, v_mem_before_reset, i_syn)``."""
        if membrane_subtract is None:
            membrane_subtract = threshold
        kind, p0, p1 = classify_surrogate(surrogate_grad_fn)
        if kind == _hip.SURR_TENSOR:
            raise ValueError("surrogate_grad_fn is not one the fused kernel can evaluate; "
                             "use LeakyIntegrator and IntegrateAndFire instead")
        check_rows_by_time("inp", inp)
        check_per_row(alpha_syn=alpha_syn, alpha_mem=alpha_mem, i_syn_init=i_syn_init, v_mem_init=v_mem_init,
                      threshold=threshold, membrane_subtract=membrane_subtract, min_v_mem=min_v_mem)
        apply_min = min_v_mem is not None
        check_parameters([alpha_mem, alpha_syn], threshold, min_v_mem)

        max_spikes = -1 if max_num_spikes_per_bin is None else int(max_num_spikes_per_bin)
        spikes, v_mem, i_syn = _hip.synLifForward(
            inp, v_mem_init, i_syn_init, alpha_mem, alpha_syn, membrane_subtract, threshold, min_v_mem,
            apply_min, max_spikes, decay_early, norm_input,
        )
        ctx.cfg = (apply_min, max_spikes, bool(decay_early), bool(norm_input), kind, p0, p1)
        ctx.set_materialize_grads(False)
        saved = [v_mem, i_syn, v_mem_init, i_syn_init, alpha_mem, alpha_syn, membrane_subtract, threshold]
        if apply_min:
            saved.append(min_v_mem)
        ctx.save_for_backward(*saved)
        return spikes, v_mem, i_syn

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_mem, grad_i_syn):
        apply_min, max_spikes, decay_early, norm_input, kind, p0, p1 = ctx.cfg
        saved = list(ctx.saved_tensors)
        v_mem, i_syn, v_mem_init, i_syn_init, alpha_mem, alpha_syn, membrane_subtract, threshold = saved[:8]
        min_v_mem = saved[8] if apply_min else None
        if grad_spikes is None and grad_v_mem is None and grad_i_syn is None:
            return (None,) * 12
        if grad_spikes is None:
            grad_spikes = torch.zeros_like(v_mem)
        if (grad_v_mem is None) != (grad_i_syn is None):
            grad_v_mem = torch.zeros_like(v_mem) if grad_v_mem is None else grad_v_mem
            grad_i_syn = torch.zeros_like(v_mem) if grad_i_syn is None else grad_i_syn
        cont = lambda x: None if x is None else x.contiguous()
        grad_input, g_am, g_as, g_v0, g_i0 = _hip.synLifBackward(
            cont(grad_spikes), cont(grad_v_mem), cont(grad_i_syn), v_mem, i_syn, v_mem_init, i_syn_init,
            alpha_mem, alpha_syn, membrane_subtract, threshold, min_v_mem, apply_min, max_spikes, decay_early,
            norm_input, kind, p0, p1,
        )
        return (grad_input, g_as, g_am, g_i0, g_v0, None, None, None, None, None, None, None)
