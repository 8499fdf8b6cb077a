"""``LeakyIntegrator``: v_t = alpha * v_{t-1} + input_t on (N, Time) matrices, as an autograd Function
on the gfx950 kernels.

Drop-in for the reference Function of the same name (reference sinabs/exodus/leaky.py:5-76): same
arguments ``(inp (N, T), alpha (N,), v_mem_init (N,))``, same checks, same three gradients.  The
backward is one fused reverse pass: input gradient ``g_t = alpha g_{t+1} + grad_t``, initial-state
gradient ``alpha g_0`` and, when ``alpha`` requires grad, ``sum_t g_t out_{t-1}`` for alpha.
"""
import torch

from . import _hip
from ._checks import check_per_row, check_rows_by_time


class LeakyIntegrator(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp: torch.Tensor, alpha: torch.Tensor, v_mem_init: torch.Tensor):
        check_rows_by_time("inp", inp)
        check_per_row(alpha=alpha, v_mem_init=v_mem_init)
        out = _hip.leakyForward(inp, v_mem_init, alpha)
        ctx.get_alpha_grads = alpha.requires_grad
        # the output is only needed again for the alpha gradient
        ctx.save_for_backward(alpha, *((out, v_mem_init) if alpha.requires_grad else ()))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        alpha, *extra = ctx.saved_tensors
        out, v_mem_init = extra if ctx.get_alpha_grads else (None, None)
        grad_input, grad_alpha, grad_init = _hip.leakyBackwardFused(
            grad_output.contiguous(), alpha, output=out, vmemInitial=v_mem_init, needAlphaGrad=ctx.get_alpha_grads
        )
        return grad_input, grad_alpha, grad_init
