"""``LeakyIntegrator`` autograd Function on the gfx950 kernels.

Same signature, checks, saved tensors and returned gradients as the reference Function
(reference sinabs/exodus/leaky.py:5-76); the backward is a single fused reverse pass that
yields the input gradient, the initial-state gradient and (when ``alpha`` requires grad) the
alpha gradient together.
"""
import torch

from . import _hip


class LeakyIntegrator(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp: torch.Tensor, alpha: torch.Tensor, v_mem_init: torch.Tensor):
        """
        Evolve a leaky integrator as ``v_t = alpha * v_{t-1} + input_t``.

        Parameters
        ----------
        inp: 2D input, shape (N, T_sim); N is anything that can be computed in parallel
            (batches, neurons...). Has to be contiguous.
        alpha: 1D, shape (N,). State decay factor exp(-dt/tau). Set 1 for IAF neurons.
        v_mem_init: 1D, shape (N,). Initial states. Has to be contiguous.
        """
        if not inp.ndim == 2:
            raise ValueError("'inp' must be 2D, (N, Time)")
        if not inp.is_contiguous():
            raise ValueError("'inp' has to be contiguous.")
        if not alpha.ndim == 1:
            raise ValueError("'alpha' must be 1D, (N,)")
        if not alpha.is_contiguous():
            raise ValueError("'alpha' has to be contiguous.")
        if not v_mem_init.ndim == 1:
            raise ValueError("'v_mem_init' must be 1D, (N,)")
        if not v_mem_init.is_contiguous():
            raise ValueError("'v_mem_init' has to be contiguous.")

        out = _hip.leakyForward(inp, v_mem_init, alpha)

        ctx.get_alpha_grads = alpha.requires_grad
        if alpha.requires_grad:
            ctx.save_for_backward(out, v_mem_init, alpha)
        else:
            ctx.save_for_backward(alpha)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        if ctx.get_alpha_grads:
            out, v_mem_init, alpha = ctx.saved_tensors
            grad_input, grad_alpha, grad_init = _hip.leakyBackwardFused(
                grad_output, alpha, output=out, vmemInitial=v_mem_init, needAlphaGrad=True
            )
        else:
            (alpha,) = ctx.saved_tensors
            grad_input, grad_alpha, grad_init = _hip.leakyBackwardFused(grad_output, alpha)
        # grad_init is one more decay step back from the first time point: alpha * grad_input[:, 0]
        return grad_input, grad_alpha, grad_init
