"""TEST INFRASTRUCTURE ONLY -- CPU checker, never imported by the shipped package.

Restatement of the *plain sinabs* way of computing the same neuron dynamics: a Python loop
over time steps made of ordinary torch operations, differentiated by torch autograd
(back-propagation through time).  This is the "reference sinabs CPU path" that the EXODUS
reference's own tests compare against (reference tests/test_spike_functions.py:198-234,
tests/test_leak_functions.py:99-124 call ``sinabs.layers.functional.lif.lif_forward``).

Upstream ``sinabs`` is a third-party dependency (``sinabs >= 1.2.9``, reference setup.py:65)
whose source is not in the reference tree and which is not installed.  The step order below
is restated from memory of that package and corroborated by the reference where it can be:
  * ``i_syn = alpha_syn * (i_syn + x)``            -- reference layers/lif.py:88-93,190-191
  * ``v = alpha * v_post + (1 - alpha) * i_syn``   -- reference layers/lif.py:206-209, cuda/lif_kernels.h:19
  * reset ``v_post = v - spikes * (subtract_value or threshold)`` -- reference layers/lif.py:237-239
  * spikes ``(v > 0) * trunc(v / theta)`` with optional cap         -- reference cuda/lif_kernels.h:20,80-81
Parity of this file with upstream sinabs is therefore UNPINNED; what is pinned is its
agreement with the mathematics (tests/test_oracle_*.py: known answers of
Gradient_analysis.ipynb cells 2, 4, 6; closed forms; the C restatement of the reference
kernels; finite differences).

``clip_mode`` selects how the lower bound is applied: ``"relu"`` is
``relu(v - lo) + lo`` (upstream's formulation as recalled), ``"max"`` is ``max(v, lo)``
(what the reference device code does, cuda/lif_kernels.h:75-77).  They agree exactly on
clipped steps and differ by at most one rounding of ``(v - lo) + lo`` on the others.  In both
modes the derivative is 0 where ``v <= lo`` (the convention of Gradient_analysis.ipynb cell 7).
"""
from __future__ import annotations

from typing import Callable, Dict, Optional, Tuple

import torch


class _ThresholdSpikes(torch.autograd.Function):
    """Spike count with a surrogate derivative: d count / d v := surrogate(v, theta)."""

    @staticmethod
    def forward(ctx, v_mem, threshold, surrogate_grad_fn, max_spikes, single):
        ctx.save_for_backward(v_mem.detach().clone())
        ctx.threshold = threshold
        ctx.surrogate_grad_fn = surrogate_grad_fn
        if single:
            return (v_mem >= threshold).float()
        counts = (v_mem > 0) * torch.div(v_mem, threshold, rounding_mode="trunc").float()
        if max_spikes is not None:
            counts = torch.clamp(counts, max=float(max_spikes))
        return counts

    @staticmethod
    def backward(ctx, grad_output):
        (v_mem,) = ctx.saved_tensors
        return grad_output * ctx.surrogate_grad_fn(v_mem, ctx.threshold), None, None, None, None


def spike_counts(v_mem, threshold, surrogate_grad_fn, max_num_spikes_per_bin: Optional[int]):
    """max_num_spikes_per_bin: None = MultiSpike, 1 = SingleSpike, k = MaxSpike(k)."""
    single = max_num_spikes_per_bin == 1
    return _ThresholdSpikes.apply(v_mem, threshold, surrogate_grad_fn, max_num_spikes_per_bin, single)


def lif_step(x_t, state: Dict[str, torch.Tensor], alpha_mem, alpha_syn, spike_threshold,
             membrane_subtract, surrogate_grad_fn, max_num_spikes_per_bin, min_v_mem, norm_input,
             spiking: bool, clip_mode: str = "relu"):
    """One time step; ``state['v_mem']`` is the post-reset potential of the previous step."""
    if alpha_syn is not None:
        i_syn = alpha_syn * (state["i_syn"] + x_t)
    else:
        i_syn = x_t
    if norm_input:
        v = alpha_mem * state["v_mem"] + (1.0 - alpha_mem) * i_syn
    else:
        v = alpha_mem * state["v_mem"] + i_syn
    if min_v_mem is not None:
        if clip_mode == "relu":
            v = torch.nn.functional.relu(v - min_v_mem) + min_v_mem
        elif clip_mode == "max":
            # value max(v, lo); derivative 0 where v <= lo (as relu gives it, and unlike
            # torch.maximum, which splits the gradient at v == lo)
            lo_t = torch.as_tensor(min_v_mem, dtype=v.dtype, device=v.device).expand_as(v)
            v = torch.where(v > lo_t, v, lo_t)
        else:
            raise ValueError(clip_mode)
    new_state = {"v_mem": v}
    if alpha_syn is not None:
        new_state["i_syn"] = i_syn
    if spiking:
        out = spike_counts(v, spike_threshold, surrogate_grad_fn, max_num_spikes_per_bin)
        sub = spike_threshold if membrane_subtract is None else membrane_subtract
        new_state["v_mem"] = v - out * sub
    else:
        out = v
    return out, v, new_state


def lif_forward(input_data, alpha_mem, alpha_syn, state: Dict[str, torch.Tensor], spike_threshold,
                membrane_subtract, surrogate_grad_fn: Optional[Callable],
                max_num_spikes_per_bin: Optional[int], min_v_mem, norm_input: bool, spiking: bool = True,
                clip_mode: str = "relu") -> Tuple[torch.Tensor, Dict[str, torch.Tensor], Dict[str, torch.Tensor]]:
    """Loop over ``input_data[:, t]`` for an input of shape (batch, time, *neurons).

    Returns (output, final state, recordings) where recordings holds the pre-reset ``v_mem``,
    the post-reset ``v_mem_post`` and, with synapses, ``i_syn``, all stacked on dim 1.
    """
    n_steps = input_data.shape[1]
    outs, v_pre, v_post, i_syn = [], [], [], []
    for t in range(n_steps):
        out, v, state = lif_step(input_data[:, t], state, alpha_mem, alpha_syn, spike_threshold,
                                 membrane_subtract, surrogate_grad_fn, max_num_spikes_per_bin, min_v_mem,
                                 norm_input, spiking, clip_mode)
        outs.append(out)
        v_pre.append(v)
        v_post.append(state["v_mem"])
        if alpha_syn is not None:
            i_syn.append(state["i_syn"])
    rec = {"v_mem": torch.stack(v_pre, 1), "v_mem_post": torch.stack(v_post, 1)}
    if alpha_syn is not None:
        rec["i_syn"] = torch.stack(i_syn, 1)
    return torch.stack(outs, 1), state, rec


def rows_to_bt(x2d: torch.Tensor, batch: int) -> torch.Tensor:
    """(batch*neurons, T) row matrix -> (batch, T, neurons)."""
    n, t = x2d.shape
    return x2d.reshape(batch, n // batch, t).movedim(-1, 1)


def bt_to_rows(x: torch.Tensor) -> torch.Tensor:
    """(batch, T, *neurons) -> contiguous (batch*neurons, T) row matrix (reference layers/lif.py:181)."""
    return x.movedim(1, -1).reshape(-1, x.shape[1]).contiguous()
