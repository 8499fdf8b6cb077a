"""TEST INFRASTRUCTURE ONLY -- CPU checker, never imported by the shipped package.

Python face of ``exodus_oracle.c`` (the scalar restatement of the reference's six device
routines) plus a restatement of the torch glue that the reference's autograd Functions wrap
around them (reference ``sinabs/exodus/spike.py:157-291`` and ``sinabs/exodus/leaky.py:43-76``).

Everything here works on CPU ``torch.float32`` tensors; the C library is reached through
``ctypes`` on ``tensor.data_ptr()``.

The surrogate-gradient callables at the bottom restate, from memory, the formulas of the
upstream ``sinabs.activation`` classes, whose source is not part of the reference tree:
their parity with upstream is UNPINNED (only ``Heaviside`` is corroborated, by the text of
``Gradient_analysis.ipynb`` cell 1).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Callable, Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libexodus_oracle.so")
_lib = None

_f32p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int


def build(force: bool = False) -> str:
    """Compile the C restatement with the committed Makefile (gcc, seconds)."""
    src = os.path.join(_HERE, "exodus_oracle.c")
    stale = not os.path.exists(_LIB_PATH) or os.path.getmtime(src) > os.path.getmtime(_LIB_PATH)
    if force or stale:
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_set_threads.argtypes = [_int]
        L.oracle_get_threads.restype = _int
        L.oracle_leaky_forward.argtypes = [_f32p] * 4 + [_i64, _i64]
        L.oracle_leaky_backward.argtypes = [_f32p] * 3 + [_i64, _i64]
        L.oracle_leaky_backward_alpha.argtypes = [_f32p] * 5 + [_i64, _i64]
        L.oracle_lif_forward.argtypes = [_f32p] * 8 + [_int, _int, _i64, _i64]
        L.oracle_lif_backward.argtypes = [_f32p] * 6 + [_i64, _i64]
        L.oracle_lif_backward_alpha.argtypes = [_f32p] * 8 + [_int, _i64, _i64]
        L.oracle_spike_forward.argtypes = [_f32p] * 2 + [ctypes.c_float] * 4 + [_int, _int, _i64, _i64]
        L.oracle_spike_backward.argtypes = [_f32p] * 4 + [ctypes.c_float] * 2 + [_i64, _i64]
        for name in ("oracle_leaky_forward", "oracle_leaky_backward", "oracle_leaky_backward_alpha",
                     "oracle_lif_forward", "oracle_lif_backward", "oracle_lif_backward_alpha",
                     "oracle_spike_forward", "oracle_spike_backward", "oracle_set_threads"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def set_threads(n: int) -> None:
    lib().oracle_set_threads(int(n))


def _chk(x: torch.Tensor, ndim: int, name: str) -> torch.Tensor:
    assert isinstance(x, torch.Tensor), name
    assert x.device.type == "cpu" and x.dtype == torch.float32, f"{name}: cpu float32 expected"
    assert x.ndim == ndim and x.is_contiguous(), f"{name}: contiguous {ndim}-D expected"
    return x


def _p(x: torch.Tensor) -> int:
    return x.data_ptr()


# --------------------------------------------------------------------------------------
# raw kernels (argument order follows the reference bindings, cuda/bindings.cu:14-257)
# --------------------------------------------------------------------------------------

def leaky_forward(inp, v_init, alpha):
    _chk(inp, 2, "inp"); _chk(v_init, 1, "v_init"); _chk(alpha, 1, "alpha")
    n, t = inp.shape
    assert v_init.numel() == n and alpha.numel() == n
    out = torch.empty_like(inp)
    lib().oracle_leaky_forward(_p(out), _p(inp), _p(v_init), _p(alpha), n, t)
    return out


def leaky_backward(grad_out, alpha):
    _chk(grad_out, 2, "grad_out"); _chk(alpha, 1, "alpha")
    n, t = grad_out.shape
    gi = torch.empty_like(grad_out)
    lib().oracle_leaky_backward(_p(gi), _p(grad_out), _p(alpha), n, t)
    return gi


def leaky_backward_alpha(grad_out, out, v_init, alpha):
    _chk(grad_out, 2, "grad_out"); _chk(out, 2, "out"); _chk(v_init, 1, "v_init"); _chk(alpha, 1, "alpha")
    n, t = grad_out.shape
    ga = torch.zeros_like(alpha)
    lib().oracle_leaky_backward_alpha(_p(ga), _p(grad_out), _p(out), _p(v_init), _p(alpha), n, t)
    return ga


def lif_forward(inp, v_init, alpha, membr_subtract, theta, theta_low, apply_theta_low, max_num_spikes):
    """Returns (spikes, v_mem) with v_mem stored before the reset of its own step."""
    _chk(inp, 2, "inp")
    n, t = inp.shape
    for nm, x in (("v_init", v_init), ("alpha", alpha), ("membr_subtract", membr_subtract), ("theta", theta)):
        _chk(x, 1, nm)
        assert x.numel() == n, nm
    if theta_low is None:
        theta_low = torch.zeros_like(theta)
    _chk(theta_low, 1, "theta_low")
    spikes = torch.empty_like(inp)
    v_mem = torch.empty_like(inp)
    lib().oracle_lif_forward(_p(spikes), _p(v_mem), _p(inp), _p(v_init), _p(alpha), _p(membr_subtract),
                             _p(theta), _p(theta_low), int(bool(apply_theta_low)), int(max_num_spikes), n, t)
    return spikes, v_mem


def lif_backward(surr, grad_out, not_clipped, alpha, csub):
    for nm, x in (("surr", surr), ("grad_out", grad_out), ("not_clipped", not_clipped)):
        _chk(x, 2, nm)
    _chk(alpha, 1, "alpha"); _chk(csub, 1, "csub")
    n, t = surr.shape
    gi = torch.empty_like(surr)
    lib().oracle_lif_backward(_p(gi), _p(grad_out), _p(surr), _p(not_clipped), _p(alpha), _p(csub), n, t)
    return gi


def lif_backward_alpha(surr, grad_out, v_post, v_post_init, not_clipped, alpha, membr_subtract,
                       gate_initial: bool = False):
    for nm, x in (("surr", surr), ("grad_out", grad_out), ("v_post", v_post), ("not_clipped", not_clipped)):
        _chk(x, 2, nm)
    n, t = surr.shape
    ga = torch.empty_like(alpha)
    lib().oracle_lif_backward_alpha(_p(ga), _p(grad_out), _p(v_post), _p(v_post_init), _p(surr),
                                    _p(not_clipped), _p(alpha), _p(membr_subtract), int(gate_initial), n, t)
    return ga


# --------------------------------------------------------------------------------------
# Function-level glue (what the reference autograd Functions compute around the kernels)
# --------------------------------------------------------------------------------------

def spike_forward(v_mem, alpha, membr_subtract, theta, theta_low, apply_theta_low, max_num_spikes):
    """Experimental spike generation; ``v_mem`` (N, T) is updated in place, returns the spikes."""
    _chk(v_mem, 2, "v_mem")
    n, t = v_mem.shape
    spikes = torch.empty_like(v_mem)
    lib().oracle_spike_forward(_p(spikes), _p(v_mem), float(alpha), float(membr_subtract), float(theta),
                               float(theta_low), int(bool(apply_theta_low)), int(max_num_spikes), n, t)
    return spikes


def spike_backward(surr, grad_out, not_clipped, alpha, membr_subtract):
    for nm, x in (("surr", surr), ("grad_out", grad_out), ("not_clipped", not_clipped)):
        _chk(x, 2, nm)
    n, t = surr.shape
    gi = torch.empty_like(surr)
    lib().oracle_spike_backward(_p(gi), _p(grad_out), _p(surr), _p(not_clipped), float(alpha),
                                float(membr_subtract), n, t)
    return gi


def integrate_and_fire_forward(inp, alpha, v_mem_init, threshold, membrane_subtract=None,
                               min_v_mem=None, max_num_spikes_per_bin: Optional[int] = None):
    """reference sinabs/exodus/spike.py:157-207 (argument checks left to the caller)."""
    if membrane_subtract is None:
        membrane_subtract = torch.ones_like(alpha) * threshold
    if min_v_mem is not None and bool((threshold <= min_v_mem).any()):
        raise ValueError("`threshold` must be greater than `min_v_mem`.")
    if bool((alpha < 0).any()) or bool((alpha > 1).any()):
        raise ValueError("'alpha' must be between 0 and 1.")
    return lif_forward(inp, v_mem_init, alpha, membrane_subtract.contiguous(), threshold, min_v_mem,
                       min_v_mem is not None, -1 if max_num_spikes_per_bin is None else max_num_spikes_per_bin)


def integrate_and_fire_backward(grad_output, grad_v_mem, v_mem, output_spikes, v_mem_init, alpha,
                                membrane_subtract, threshold, min_v_mem, surrogate_grad_fn: Callable,
                                need_alpha_grad: bool, gate_initial: bool = False
                                ) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
    """reference sinabs/exodus/spike.py:250-291; returns (grad_input, grad_alpha|None, grad_init)."""
    surrogates = surrogate_grad_fn(v_mem, threshold.unsqueeze(1)).contiguous()
    if min_v_mem is not None:
        not_clipped = (v_mem > min_v_mem.unsqueeze(1)).float()
    else:
        not_clipped = torch.ones_like(surrogates)
    if grad_v_mem is None:
        grad_v_mem = torch.zeros_like(v_mem)
    if grad_output is None:
        grad_output = torch.zeros_like(v_mem)
    g = (surrogates * grad_output + grad_v_mem).contiguous()
    grad_input = lif_backward(surrogates, g, not_clipped, alpha, (alpha * membrane_subtract).contiguous())
    grad_alpha = None
    if need_alpha_grad:
        v_post = (v_mem - membrane_subtract.unsqueeze(1) * output_spikes).contiguous()
        grad_alpha = lif_backward_alpha(surrogates, g, v_post, v_mem_init, not_clipped, alpha,
                                        membrane_subtract, gate_initial=gate_initial)
    grad_init = alpha * grad_input[:, 0]
    return grad_input, grad_alpha, grad_init


def leaky_integrator_backward(grad_output, out, v_mem_init, alpha, need_alpha_grad: bool):
    """reference sinabs/exodus/leaky.py:53-76; returns (grad_input, grad_alpha|None, grad_init)."""
    grad_alpha = leaky_backward_alpha(grad_output, out, v_mem_init, alpha) if need_alpha_grad else None
    grad_input = leaky_backward(grad_output, alpha)
    return grad_input, grad_alpha, alpha * grad_input[:, 0]


# --------------------------------------------------------------------------------------
# linear-time reverse recurrence in float64 (independent statement of the same gradient)
# --------------------------------------------------------------------------------------

def lif_backward_recurrence_f64(surr, g, not_clipped, alpha, membrane_subtract, v_post=None, v_post_init=None):
    """lambda_t = nc_t (g_t + alpha (1 - c s_t) lambda_{t+1}); grad_alpha = sum_t lambda_t vpost_{t-1}.

    Algebraically equal to the quadratic sum of reference cuda/lif_kernels.h:105-107 and to the exact
    (initial-step-gated) form of :179-182.  Returns float64 (grad_input, grad_alpha|None, grad_init).
    """
    s = surr.double(); gg = g.double(); nc = not_clipped.double()
    a = alpha.double(); c = membrane_subtract.double()
    n, t = s.shape
    lam = torch.zeros(n, dtype=torch.float64)
    gi = torch.empty_like(s)
    ga = torch.zeros(n, dtype=torch.float64) if v_post is not None else None
    for k in range(t - 1, -1, -1):
        lam = nc[:, k] * (gg[:, k] + a * (1.0 - c * s[:, k]) * lam)
        gi[:, k] = lam
        if ga is not None:
            prev = v_post[:, k - 1].double() if k > 0 else v_post_init.double()
            ga += lam * prev
    return gi, ga, a * gi[:, 0]


# --------------------------------------------------------------------------------------
# surrogate gradients  (formulas recalled from upstream sinabs.activation -- UNPINNED)
# --------------------------------------------------------------------------------------

class Heaviside:
    """1/theta where v_mem >= theta - window, else 0 (Gradient_analysis.ipynb cell 1)."""

    def __init__(self, window: float = 1.0):
        self.window = window

    def __call__(self, v_mem, threshold):
        return (v_mem >= (threshold - self.window)).float() / threshold


class SingleExponential:
    """scale / (theta w) * exp(-|v - theta| / (theta w))."""

    def __init__(self, grad_width: float = 0.5, grad_scale: float = 1.0):
        self.grad_width, self.grad_scale = grad_width, grad_scale

    def __call__(self, v_mem, threshold):
        width = threshold * self.grad_width
        return self.grad_scale / width * torch.exp(-torch.abs(v_mem - threshold) / width)


class PeriodicExponential:
    """Exponential bump around theta, repeated with period theta above theta.

    u = v - theta/2; for v >= theta, u is wrapped into [0, theta); result =
    scale * exp(-|u - theta/2| / w) / theta.
    """

    def __init__(self, grad_width: float = 0.5, grad_scale: float = 1.0):
        self.grad_width, self.grad_scale = grad_width, grad_scale

    def __call__(self, v_mem, threshold):
        shifted = v_mem - threshold / 2
        periodic = torch.remainder(shifted, threshold)
        u = torch.where(v_mem >= threshold, periodic, shifted)
        return self.grad_scale * torch.exp(-torch.abs(u - threshold / 2) / self.grad_width) / threshold
