"""``IntegrateAndFire`` autograd Function on the gfx950 kernels.

Keeps the reference's signature, argument checks and error messages
(reference sinabs/exodus/spike.py:107-291).  What differs is where the work happens:

* forward: one kernel writes spikes and pre-reset membrane potential in a single pass;
* backward: one reverse pass over the saved membrane potential produces the input gradient,
  the initial-state gradient and the alpha gradient.  Surrogate gradient, clip mask, spike
  counts and post-reset potential are recomputed in registers from ``v_mem`` instead of being
  materialised as (N, T) tensors.  The linear-time recurrence
  ``lambda_t = nc_t (g_t + alpha (1 - c s_t) lambda_{t+1})`` replaces the reference's
  quadratic sum (reference cuda/lif_kernels.h:105-107,147-166); both define the same vector.

Surrogate functions known to the kernels (the ``sinabs.activation`` classes
``SingleExponential``, ``PeriodicExponential`` and ``Heaviside``) are evaluated in-kernel; any
other callable is evaluated with torch on the device, as the reference does
(reference sinabs/exodus/spike.py:251), and handed to the same kernel as a tensor.
"""
from typing import Callable, Optional, Tuple, Union

import torch

from . import _hip, hbm
from ._checks import check_per_row, check_rows_by_time
from ._validate import check_parameters

_KNOWN_SURROGATE_MODULES = ("sinabs.activation", "sinabs.exodus._compat")


def classify_surrogate(fn) -> Tuple[int, float, float]:
    """Map a surrogate-gradient callable to (kernel kind, p0, p1); kind 0 = evaluate with torch."""
    cls = type(fn)
    mod = getattr(cls, "__module__", "") or ""
    if not mod.startswith(_KNOWN_SURROGATE_MODULES):
        return _hip.SURR_TENSOR, 0.0, 0.0
    name = cls.__name__
    try:
        if name == "SingleExponential":
            return _hip.SURR_SINGLE_EXP, float(fn.grad_width), float(fn.grad_scale)
        if name == "PeriodicExponential":
            return _hip.SURR_PERIODIC_EXP, float(fn.grad_width), float(fn.grad_scale)
        if name == "Heaviside":
            return _hip.SURR_HEAVISIDE, float(fn.window), 0.0
    except (AttributeError, TypeError, ValueError):
        pass
    return _hip.SURR_TENSOR, 0.0, 0.0


class IntegrateAndFire(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        inp: torch.Tensor,
        alpha: torch.Tensor,
        v_mem_init: torch.Tensor,
        threshold: torch.Tensor,
        membrane_subtract: torch.Tensor,
        min_v_mem: Union[torch.Tensor, None],
        surrogate_grad_fn: Callable,
        max_num_spikes_per_bin: Optional[int] = None,
    ):
        """
        Integrate membrane potential with or without leak, generate spikes and apply the
        subtractive reset.

        Parameters
        ----------
        inp: (N, T_sim) contiguous input; N is anything that can be computed in parallel.
        alpha: (N,) state decay factor exp(-dt/tau); 1 for IAF neurons.
        v_mem_init: (N,) initial membrane potential (after reset).
        threshold: (N,) firing thresholds.
        membrane_subtract: (N,) value subtracted per spike; None = threshold.
        min_v_mem: (N,) lower limits for v_mem, or None for no limit.
        surrogate_grad_fn: callable (v_mem, threshold) -> d spikes / d v_mem.
        max_num_spikes_per_bin: cap on spikes per step; None removes the limit.

        Returns
        -------
        (output_spikes, v_mem), both (N, T_sim); v_mem is the potential before reset.
        """
        if membrane_subtract is None:
            membrane_subtract = torch.ones_like(alpha) * threshold
        apply_min_v_mem = min_v_mem is not None

        check_rows_by_time("inp", inp)
        check_per_row(alpha=alpha, membrane_subtract=membrane_subtract, v_mem_init=v_mem_init, threshold=threshold,
                      min_v_mem=min_v_mem)

        check_parameters([alpha], threshold, min_v_mem)      # alpha in [0, 1], threshold > min_v_mem

        v_mem = hbm.empty_like(inp)                # after hbm.enable(): in memory striped over the regions of HBM
        output_spikes = hbm.empty_like(inp)
        max_spikes = -1 if max_num_spikes_per_bin is None else int(max_num_spikes_per_bin)

        _hip.lifForward(
            output_spikes, v_mem, inp, v_mem_init, alpha, membrane_subtract, threshold,
            min_v_mem, apply_min_v_mem, max_spikes,
        )

        ctx.surrogate_grad_fn = surrogate_grad_fn
        ctx.apply_min_v_mem = apply_min_v_mem
        ctx.max_spikes = max_spikes
        ctx.get_alpha_grads = alpha.requires_grad
        ctx.set_materialize_grads(False)
        # v_mem is stored before reset (surrogate gradients are functions of it); the spike
        # raster is not saved: the backward kernel recomputes counts from v_mem.
        saved = [v_mem, alpha, membrane_subtract, threshold]
        if apply_min_v_mem:
            saved.append(min_v_mem)
        if alpha.requires_grad:
            saved.append(v_mem_init)
        ctx.save_for_backward(*saved)

        return output_spikes, v_mem

    @staticmethod
    def backward(ctx, grad_output, grad_v_mem):
        saved = list(ctx.saved_tensors)
        v_mem, alpha, membrane_subtract, threshold = saved[:4]
        rest = saved[4:]
        min_v_mem = rest.pop(0) if ctx.apply_min_v_mem else None
        v_mem_init = rest.pop(0) if ctx.get_alpha_grads else None

        if grad_output is None and grad_v_mem is None:
            return (None,) * 8
        if grad_output is None:
            grad_output = torch.zeros_like(v_mem)
        grad_output = grad_output.contiguous()
        if grad_v_mem is not None:
            grad_v_mem = grad_v_mem.contiguous()

        kind, p0, p1 = classify_surrogate(ctx.surrogate_grad_fn)
        surrogates = None
        if kind == _hip.SURR_TENSOR:
            surrogates = ctx.surrogate_grad_fn(v_mem, threshold.unsqueeze(1)).float().contiguous()

        grad_input, grad_alpha, grad_init = _hip.lifBackwardFused(
            grad_output, grad_v_mem, v_mem, v_mem_init, alpha, membrane_subtract, threshold, min_v_mem,
            ctx.apply_min_v_mem, ctx.max_spikes, kind, p0, p1, surr=surrogates,
            needAlphaGrad=ctx.get_alpha_grads,
        )
        # grad_init back-propagates one more decay step from the first time point
        # (d v_0 / d v_init = alpha, the reset on v_init is applied by the caller).
        return (grad_input, grad_alpha, grad_init, None, None, None, None, None)


class SpikeFunction(torch.autograd.Function):
    """Experimental: spikes from a membrane potential that already contains the response to the
    input; resets and lower bound are applied to ``v_mem`` in place
    (reference sinabs/exodus/spike.py:7-104).  ``IntegrateAndFire`` is the faster option.

    Arguments as in the reference: ``v_mem`` (N, T) contiguous, scalar ``membrane_subtract``,
    ``alpha``, ``threshold``, optional scalar ``min_v_mem``, optional ``max_num_spikes_per_bin``.
    Returns ``(spikes, v_mem)``.  One deliberate difference: the reference hands ``threshold``
    to the kernel where the lower bound belongs (spike.py:63); here ``min_v_mem`` is the bound.
    """

    @staticmethod
    def forward(
        ctx,
        v_mem: torch.Tensor,
        membrane_subtract: float,
        alpha: float,
        surrogate_grad_fn: Callable,
        threshold: float,
        min_v_mem: Optional[float] = None,
        max_num_spikes_per_bin: Optional[int] = None,
    ):
        if not v_mem.is_contiguous():
            raise ValueError("'v_mem' has to be contiguous.")
        if not v_mem.ndim == 2:
            raise ValueError("'v_mem' must be 2D, (N, Time)")
        scalar = lambda v: float(v.item()) if isinstance(v, torch.Tensor) else float(v)
        threshold, alpha, membrane_subtract = scalar(threshold), scalar(alpha), scalar(membrane_subtract)
        min_v_mem = None if min_v_mem is None else scalar(min_v_mem)
        if min_v_mem is not None and threshold <= min_v_mem:
            raise ValueError("`threshold` must be greater than `min_v_mem`.")

        spikes = _hip.spikeForward(
            v_mem, alpha, membrane_subtract, threshold,
            0.0 if min_v_mem is None else min_v_mem,
            min_v_mem is not None,
            -1 if max_num_spikes_per_bin is None else max_num_spikes_per_bin,
        )
        ctx.alpha = alpha
        ctx.threshold = threshold
        ctx.min_v_mem = min_v_mem
        ctx.membrane_subtract = membrane_subtract
        ctx.surrogate_grad_fn = surrogate_grad_fn
        ctx.save_for_backward(v_mem)
        return spikes, v_mem

    @staticmethod
    def backward(ctx, grad_output, grad_v_mem):
        if grad_v_mem is not None and torch.count_nonzero(grad_v_mem) > 0:
            raise NotImplementedError(
                "Direct Backpropagation through membrane potential is currently not supported."
            )
        (v_mem,) = ctx.saved_tensors
        surrogates = ctx.surrogate_grad_fn(v_mem, ctx.threshold)
        if ctx.min_v_mem is None:
            not_clipped = torch.ones_like(surrogates)
        else:
            not_clipped = (v_mem > ctx.min_v_mem).float()
        grad_input = _hip.spikeBackward(
            surrogates.contiguous(), grad_output.contiguous(), not_clipped.contiguous(),
            ctx.alpha, ctx.membrane_subtract,
        )
        return grad_input, None, None, None, None, None, None
