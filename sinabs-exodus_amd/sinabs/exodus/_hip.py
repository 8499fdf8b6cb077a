"""ctypes loader for ``libexodus_hip.so`` and thin tensor-level wrappers around its C ABI.

This module plays the role of the reference's ``exodus_cuda`` pybind module
(reference cuda/bindings.cu:362-373): same six functions, same argument order, plus the two
fused backward entry points.  Tensors must live on a HIP device, be ``float32`` and contiguous;
anything else raises, as the reference's ``CHECK_INPUT`` asserts do
(reference cuda/bindings.cu:7-10).  There is no CPU path: if the shared library is missing the
import of this module fails with an ``ImportError`` that says how to build it.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional

import torch  # must be imported before the library so both share one HIP runtime

from . import hbm

_HERE = os.path.dirname(os.path.abspath(__file__))
# EXODUS_HIP_LIBRARY may point at another build of the same ABI (e.g. one compiled with other flags)
LIB_PATH = os.environ.get("EXODUS_HIP_LIBRARY") or os.path.join(_HERE, "libexodus_hip.so")

SURR_TENSOR, SURR_SINGLE_EXP, SURR_PERIODIC_EXP, SURR_HEAVISIDE = 0, 1, 2, 3
ABI_VERSION = 8

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f = ctypes.c_float

_SIGNATURES = {
    "exodus_hip_abi_version": ([], _int),
    "exodus_hip_error_string": ([_int], ctypes.c_char_p),
    "exodus_lif_forward": ([_p] * 8 + [_int, _int, _i64, _i64, _p], _int),
    "exodus_lif_backward": ([_p] * 6 + [_i64, _i64, _p], _int),
    "exodus_lif_backward_alpha": ([_p] * 8 + [_int, _i64, _i64, _p], _int),
    "exodus_leaky_forward": ([_p] * 4 + [_i64, _i64, _p], _int),
    "exodus_leaky_backward": ([_p] * 3 + [_i64, _i64, _p], _int),
    "exodus_leaky_backward_alpha": ([_p] * 5 + [_i64, _i64, _p], _int),
    "exodus_leaky_backward_fused": ([_p] * 7 + [_i64, _i64, _p], _int),
    "exodus_lif_backward_fused": ([_p] * 12 + [_int, _int, _int, _f, _f, _i64, _i64, _p], _int),
    "exodus_synlif_forward": ([_p] * 11 + [_int, _int, _int, _int, _i64, _i64, _p], _int),
    "exodus_synlif_backward": ([_p] * 17 + [_int, _int, _int, _int, _int, _f, _f, _i64, _i64, _p], _int),
    "exodus_spike_forward": ([_p, _p, _f, _f, _f, _f, _int, _int, _i64, _i64, _p], _int),
    "exodus_spike_backward": ([_p] * 4 + [_f, _f, _i64, _i64, _p], _int),
    "exodus_layer_checkpoint_interval": ([], _int),
    "exodus_layer_lif_forward": ([_p] * 16 + [_int, _int, _int, _int, _int, _i64, _i64, _i64, _p], _int),
    "exodus_layer_lif_backward": ([_p] * 18 + [_int, _int, _int, _int, _int, _f, _f, _p, _p, _p, _int, _i64, _i64, _i64, _p], _int),
    "exodus_layer_backward_time_split": ([_int], _int),
    "exodus_layer_scratch_floats": ([], _i64),
    "exodus_layer_lif_backward_from_input": ([_p] * 16 + [_int, _int, _int, _int, _int, _f, _f, _p, _p, _p, _int, _i64, _i64, _i64, _p], _int),
    "exodus_layer_leaky_forward": ([_p] * 6 + [_int, _int, _i64, _i64, _i64, _p], _int),
    "exodus_layer_leaky_backward": ([_p] * 9 + [_int, _int, _int, _i64, _i64, _i64, _p], _int),
    "exodus_hbm_regions_create": ([_int, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, _int, ctypes.c_uint64, _p], _int),
    "exodus_hbm_regions_destroy": ([_int], _int),
    "exodus_hbm_alloc_striped": ([ctypes.c_size_t, _int, _p], _p),
    "exodus_hbm_alloc_region0": ([ctypes.c_size_t, _int, _p], _p),
    "exodus_hbm_alloc_region1": ([ctypes.c_size_t, _int, _p], _p),
    "exodus_hbm_alloc_region2": ([ctypes.c_size_t, _int, _p], _p),
    "exodus_hbm_free": ([_p, ctypes.c_size_t, _int, _p], None),
    "exodus_hbm_usage": ([_int, _p, _p], _int),
}


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found. Build it with `python build_hip.py` in the package root "
            "(needs hipcc; cross-compiles for gfx950 without a GPU). There is no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (argtypes, restype) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = library/header mismatch
        fn.argtypes = argtypes
        fn.restype = restype
    got = lib.exodus_hip_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"libexodus_hip.so has ABI version {got}, this package expects {ABI_VERSION}")
    return lib


lib = _load()


class ExodusHipError(RuntimeError):
    pass


def _check(status: int, what: str) -> None:
    if status != 0:
        msg = lib.exodus_hip_error_string(status)
        raise ExodusHipError(f"{what} failed: {msg.decode() if msg else status} (status {status})")


def _dev(x: torch.Tensor, name: str, like: Optional[torch.Tensor] = None) -> torch.Tensor:
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a tensor on a HIP device (got {x.device}); there is no CPU path")
    if x.dtype != torch.float32:
        raise RuntimeError(f"{name} must be float32 (got {x.dtype})")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if like is not None and x.device != like.device:
        raise RuntimeError(f"{name} and the first tensor must be on the same device")
    return x


def _rows(x: torch.Tensor, name: str, n: int) -> torch.Tensor:
    if x.ndim != 1 or x.shape[0] != n:
        raise RuntimeError(f"{name} must have shape ({n},), got {tuple(x.shape)}")
    return x


def _mat(x: torch.Tensor, name: str, n: int, t: int) -> torch.Tensor:
    if x.ndim != 2 or x.shape[0] != n or x.shape[1] != t:
        raise RuntimeError(f"{name} must have shape ({n}, {t}), got {tuple(x.shape)}")
    return x


def _ptr(x: Optional[torch.Tensor]):
    return None if x is None else x.data_ptr()             # ctypes takes a plain integer for a void pointer


def _stream(x: torch.Tensor):
    return torch.cuda.current_stream(x.device).cuda_stream or None


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on_device_of(device: torch.device):
    """Device guard for a launch: ``device`` becomes current for the call -- which it nearly always is already, and
    then nothing needs switching."""
    return _NO_GUARD if torch.cuda.current_device() == device.index else torch.cuda.device(device)


# ------------------------------------------------------------------------------------------
# the six functions of the reference extension, same names and argument order
# ------------------------------------------------------------------------------------------

def lifForward(outputSpikes, vmem, input, vmemPostInitial, alpha, membrSubtract, theta, thetaLow,
               applyThetaLow: bool, maxNumSpikes: int) -> None:
    """reference cuda/bindings.cu:14-70; fills the caller-allocated ``outputSpikes`` and ``vmem``."""
    _dev(input, "input")
    if input.ndim != 2:
        raise RuntimeError("input must be 2-D (rows, time)")
    n, t = input.shape
    _mat(_dev(outputSpikes, "outputSpikes", input), "outputSpikes", n, t)
    _mat(_dev(vmem, "vmem", input), "vmem", n, t)
    for nm, x in (("vmemPostInitial", vmemPostInitial), ("alpha", alpha), ("membrSubtract", membrSubtract),
                  ("theta", theta)):
        _rows(_dev(x, nm, input), nm, n)
    if applyThetaLow:
        _rows(_dev(thetaLow, "thetaLow", input), "thetaLow", n)
    else:
        thetaLow = None
    with _on_device_of(input.device):
        _check(lib.exodus_lif_forward(_ptr(outputSpikes), _ptr(vmem), _ptr(input), _ptr(vmemPostInitial),
                                      _ptr(alpha), _ptr(membrSubtract), _ptr(theta), _ptr(thetaLow),
                                      int(bool(applyThetaLow)), int(maxNumSpikes), n, t, _stream(input)),
               "exodus_lif_forward")


def lifBackward(surr, outputGrad, notClipped, alpha, membrSubtract) -> torch.Tensor:
    """reference cuda/bindings.cu:72-110; ``membrSubtract`` is alpha times the subtract value."""
    _dev(surr, "surr")
    if surr.ndim != 2:
        raise RuntimeError("surr must be 2-D (rows, time)")
    n, t = surr.shape
    _mat(_dev(outputGrad, "outputGrad", surr), "outputGrad", n, t)
    _mat(_dev(notClipped, "notClipped", surr), "notClipped", n, t)
    _rows(_dev(alpha, "alpha", surr), "alpha", n)
    _rows(_dev(membrSubtract, "membrSubtract", surr), "membrSubtract", n)
    inputGrad = hbm.empty_like(surr)
    with _on_device_of(surr.device):
        _check(lib.exodus_lif_backward(_ptr(inputGrad), _ptr(surr), _ptr(outputGrad), _ptr(notClipped),
                                       _ptr(alpha), _ptr(membrSubtract), n, t, _stream(surr)),
               "exodus_lif_backward")
    return inputGrad


def lifBackwardAlpha(surr, outputGrad, vmemPost, vmemPostInitial, notClipped, alpha, membrSubtract,
                     gateInitial: bool = False) -> torch.Tensor:
    """reference cuda/bindings.cu:112-158.  ``gateInitial=False`` is the reference's arithmetic."""
    _dev(surr, "surr")
    if surr.ndim != 2:
        raise RuntimeError("surr must be 2-D (rows, time)")
    n, t = surr.shape
    for nm, x in (("outputGrad", outputGrad), ("vmemPost", vmemPost), ("notClipped", notClipped)):
        _mat(_dev(x, nm, surr), nm, n, t)
    for nm, x in (("vmemPostInitial", vmemPostInitial), ("alpha", alpha), ("membrSubtract", membrSubtract)):
        _rows(_dev(x, nm, surr), nm, n)
    alphaGrad = torch.zeros_like(alpha)
    with _on_device_of(surr.device):
        _check(lib.exodus_lif_backward_alpha(_ptr(alphaGrad), _ptr(surr), _ptr(outputGrad), _ptr(vmemPost),
                                             _ptr(vmemPostInitial), _ptr(notClipped), _ptr(alpha),
                                             _ptr(membrSubtract), int(bool(gateInitial)), n, t, _stream(surr)),
               "exodus_lif_backward_alpha")
    return alphaGrad


def leakyForward(input, vmemInitial, alpha, *, output=None) -> torch.Tensor:
    """reference cuda/bindings.cu:163-193.  ``output`` (not in the reference) is a preallocated result."""
    _dev(input, "input")
    if input.ndim != 2:
        raise RuntimeError("input must be 2-D (rows, time)")
    n, t = input.shape
    _rows(_dev(vmemInitial, "vmemInitial", input), "vmemInitial", n)
    _rows(_dev(alpha, "alpha", input), "alpha", n)
    out = hbm.empty_like(input) if output is None else _mat(_dev(output, "output", input), "output", n, t)
    with _on_device_of(input.device):
        _check(lib.exodus_leaky_forward(_ptr(out), _ptr(input), _ptr(vmemInitial), _ptr(alpha), n, t,
                                        _stream(input)), "exodus_leaky_forward")
    return out


def leakyBackward(outputGrad, alpha) -> torch.Tensor:
    """reference cuda/bindings.cu:195-221."""
    _dev(outputGrad, "outputGrad")
    if outputGrad.ndim != 2:
        raise RuntimeError("outputGrad must be 2-D (rows, time)")
    n, t = outputGrad.shape
    _rows(_dev(alpha, "alpha", outputGrad), "alpha", n)
    inputGrad = hbm.empty_like(outputGrad)
    with _on_device_of(outputGrad.device):
        _check(lib.exodus_leaky_backward(_ptr(inputGrad), _ptr(outputGrad), _ptr(alpha), n, t,
                                         _stream(outputGrad)), "exodus_leaky_backward")
    return inputGrad


def leakyBackwardAlpha(outputGrad, output, vmemInitial, alpha) -> torch.Tensor:
    """reference cuda/bindings.cu:223-257."""
    _dev(outputGrad, "outputGrad")
    if outputGrad.ndim != 2:
        raise RuntimeError("outputGrad must be 2-D (rows, time)")
    n, t = outputGrad.shape
    _mat(_dev(output, "output", outputGrad), "output", n, t)
    _rows(_dev(vmemInitial, "vmemInitial", outputGrad), "vmemInitial", n)
    _rows(_dev(alpha, "alpha", outputGrad), "alpha", n)
    alphaGrad = torch.zeros_like(alpha)
    with _on_device_of(outputGrad.device):
        _check(lib.exodus_leaky_backward_alpha(_ptr(alphaGrad), _ptr(outputGrad), _ptr(output),
                                               _ptr(vmemInitial), _ptr(alpha), n, t, _stream(outputGrad)),
               "exodus_leaky_backward_alpha")
    return alphaGrad


def spikeForward(vmem, alpha: float, membrSubtract: float, theta: float, thetaLow: float, applyThetaLow: bool,
                 maxNumSpikes: int) -> torch.Tensor:
    """reference cuda/bindings.cu:262-290 (experimental): ``vmem`` (rows, time) is corrected in place
    for resets and lower bound, the spike raster is returned."""
    _dev(vmem, "vmem")
    if vmem.ndim != 2:
        raise RuntimeError("vmem must be 2-D (rows, time)")
    n, t = vmem.shape
    spikes = hbm.empty_like(vmem)
    with _on_device_of(vmem.device):
        _check(lib.exodus_spike_forward(_ptr(spikes), _ptr(vmem), float(alpha), float(membrSubtract), float(theta),
                                        float(thetaLow), int(bool(applyThetaLow)), int(maxNumSpikes), n, t,
                                        _stream(vmem)), "exodus_spike_forward")
    return spikes


def spikeBackward(surr, outputGrad, notClipped, alpha: float, membrSubtract: float) -> torch.Tensor:
    """reference cuda/bindings.cu:327-359 (experimental)."""
    _dev(surr, "surr")
    if surr.ndim != 2:
        raise RuntimeError("surr must be 2-D (rows, time)")
    n, t = surr.shape
    _mat(_dev(outputGrad, "outputGrad", surr), "outputGrad", n, t)
    _mat(_dev(notClipped, "notClipped", surr), "notClipped", n, t)
    inputGrad = hbm.empty_like(surr)
    with _on_device_of(surr.device):
        _check(lib.exodus_spike_backward(_ptr(inputGrad), _ptr(surr), _ptr(outputGrad), _ptr(notClipped),
                                         float(alpha), float(membrSubtract), n, t, _stream(surr)),
               "exodus_spike_backward")
    return inputGrad


# ------------------------------------------------------------------------------------------
# fused backward passes (what the autograd Functions use)
# ------------------------------------------------------------------------------------------

def leakyBackwardFused(outputGrad, alpha, output=None, vmemInitial=None, needAlphaGrad: bool = False,
                       inputGrad: Optional[torch.Tensor] = None):
    """One reverse pass: returns (inputGrad, alphaGrad | None, initGrad)."""
    _dev(outputGrad, "outputGrad")
    if outputGrad.ndim != 2:
        raise RuntimeError("outputGrad must be 2-D (rows, time)")
    n, t = outputGrad.shape
    _rows(_dev(alpha, "alpha", outputGrad), "alpha", n)
    if needAlphaGrad:
        _mat(_dev(output, "output", outputGrad), "output", n, t)
        _rows(_dev(vmemInitial, "vmemInitial", outputGrad), "vmemInitial", n)
    if inputGrad is None:
        inputGrad = hbm.empty_like(outputGrad)
    else:
        _mat(_dev(inputGrad, "inputGrad", outputGrad), "inputGrad", n, t)
    initGrad = torch.zeros_like(alpha)
    alphaGrad = torch.zeros_like(alpha) if needAlphaGrad else None
    with _on_device_of(outputGrad.device):
        _check(lib.exodus_leaky_backward_fused(_ptr(inputGrad), _ptr(alphaGrad), _ptr(initGrad), _ptr(outputGrad),
                                               _ptr(output) if needAlphaGrad else None,
                                               _ptr(vmemInitial) if needAlphaGrad else None, _ptr(alpha), n, t,
                                               _stream(outputGrad)), "exodus_leaky_backward_fused")
    return inputGrad, alphaGrad, initGrad


def lifBackwardFused(gradSpikes, gradVmem, vmem, vmemPostInitial, alpha, membrSubtract, theta, thetaLow,
                     applyThetaLow: bool, maxNumSpikes: int, surrogateKind: int, surrP0: float = 0.0,
                     surrP1: float = 0.0, surr: Optional[torch.Tensor] = None, needAlphaGrad: bool = False,
                     inputGrad: Optional[torch.Tensor] = None):
    """One reverse pass over the saved membrane potential: returns (inputGrad, alphaGrad | None, initGrad).

    ``membrSubtract`` is the plain subtract value here (not pre-multiplied by alpha).
    """
    _dev(vmem, "vmem")
    if vmem.ndim != 2:
        raise RuntimeError("vmem must be 2-D (rows, time)")
    n, t = vmem.shape
    _mat(_dev(gradSpikes, "gradSpikes", vmem), "gradSpikes", n, t)
    if gradVmem is not None:
        _mat(_dev(gradVmem, "gradVmem", vmem), "gradVmem", n, t)
    for nm, x in (("alpha", alpha), ("membrSubtract", membrSubtract), ("theta", theta)):
        _rows(_dev(x, nm, vmem), nm, n)
    if applyThetaLow:
        _rows(_dev(thetaLow, "thetaLow", vmem), "thetaLow", n)
    else:
        thetaLow = None
    if needAlphaGrad:
        _rows(_dev(vmemPostInitial, "vmemPostInitial", vmem), "vmemPostInitial", n)
    if surrogateKind == SURR_TENSOR:
        _mat(_dev(surr, "surr", vmem), "surr", n, t)
    else:
        surr = None
    if inputGrad is None:
        inputGrad = hbm.empty_like(vmem)
    else:
        _mat(_dev(inputGrad, "inputGrad", vmem), "inputGrad", n, t)
    initGrad = torch.zeros_like(alpha)
    alphaGrad = torch.zeros_like(alpha) if needAlphaGrad else None
    with _on_device_of(vmem.device):
        _check(lib.exodus_lif_backward_fused(_ptr(inputGrad), _ptr(alphaGrad), _ptr(initGrad), _ptr(gradSpikes),
                                             _ptr(gradVmem), _ptr(vmem), _ptr(surr),
                                             _ptr(vmemPostInitial) if needAlphaGrad else None, _ptr(alpha),
                                             _ptr(membrSubtract), _ptr(theta), _ptr(thetaLow),
                                             int(bool(applyThetaLow)), int(maxNumSpikes), int(surrogateKind),
                                             float(surrP0), float(surrP1), n, t, _stream(vmem)),
               "exodus_lif_backward_fused")
    return inputGrad, alphaGrad, initGrad


def synLifForward(input, vmemPostInitial, isynInitial, alphaMem, alphaSyn, membrSubtract, theta, thetaLow,
                  applyThetaLow: bool, maxNumSpikes: int, decayEarly: bool, normInput: bool,
                  out: Optional[tuple] = None):
    """Fused synapse + membrane forward: returns (spikes, vmem, isyn), all (n, t)."""
    _dev(input, "input")
    if input.ndim != 2:
        raise RuntimeError("input must be 2-D (rows, time)")
    n, t = input.shape
    for nm, x in (("vmemPostInitial", vmemPostInitial), ("isynInitial", isynInitial), ("alphaMem", alphaMem),
                  ("alphaSyn", alphaSyn), ("membrSubtract", membrSubtract), ("theta", theta)):
        _rows(_dev(x, nm, input), nm, n)
    if applyThetaLow:
        _rows(_dev(thetaLow, "thetaLow", input), "thetaLow", n)
    else:
        thetaLow = None
    if out is None:
        out = (hbm.empty_like(input), hbm.empty_like(input), hbm.empty_like(input))
    spikes, vmem, isyn = out
    for nm, x in (("spikes", spikes), ("vmem", vmem), ("isyn", isyn)):
        _mat(_dev(x, nm, input), nm, n, t)
    with _on_device_of(input.device):
        _check(lib.exodus_synlif_forward(_ptr(spikes), _ptr(vmem), _ptr(isyn), _ptr(input), _ptr(vmemPostInitial),
                                         _ptr(isynInitial), _ptr(alphaMem), _ptr(alphaSyn), _ptr(membrSubtract),
                                         _ptr(theta), _ptr(thetaLow), int(bool(applyThetaLow)), int(maxNumSpikes),
                                         int(bool(decayEarly)), int(bool(normInput)), n, t, _stream(input)),
               "exodus_synlif_forward")
    return spikes, vmem, isyn


def synLifBackward(gradSpikes, gradVmem, gradIsyn, vmem, isyn, vmemPostInitial, isynInitial, alphaMem, alphaSyn,
                   membrSubtract, theta, thetaLow, applyThetaLow: bool, maxNumSpikes: int, decayEarly: bool,
                   normInput: bool, surrogateKind: int, surrP0: float, surrP1: float,
                   inputGrad: Optional[torch.Tensor] = None):
    """Fused reverse pass: returns (inputGrad, alphaMemGrad, alphaSynGrad, vmemInitGrad, isynInitGrad)."""
    _dev(vmem, "vmem")
    if vmem.ndim != 2:
        raise RuntimeError("vmem must be 2-D (rows, time)")
    n, t = vmem.shape
    _mat(_dev(gradSpikes, "gradSpikes", vmem), "gradSpikes", n, t)
    _mat(_dev(isyn, "isyn", vmem), "isyn", n, t)
    if (gradVmem is None) != (gradIsyn is None):
        raise RuntimeError("gradVmem and gradIsyn must be given together")
    if gradVmem is not None:
        _mat(_dev(gradVmem, "gradVmem", vmem), "gradVmem", n, t)
        _mat(_dev(gradIsyn, "gradIsyn", vmem), "gradIsyn", n, t)
    for nm, x in (("vmemPostInitial", vmemPostInitial), ("isynInitial", isynInitial), ("alphaMem", alphaMem),
                  ("alphaSyn", alphaSyn), ("membrSubtract", membrSubtract), ("theta", theta)):
        _rows(_dev(x, nm, vmem), nm, n)
    if applyThetaLow:
        _rows(_dev(thetaLow, "thetaLow", vmem), "thetaLow", n)
    else:
        thetaLow = None
    if inputGrad is None:
        inputGrad = hbm.empty_like(vmem)
    else:
        _mat(_dev(inputGrad, "inputGrad", vmem), "inputGrad", n, t)
    per_row = [torch.zeros_like(alphaMem) for _ in range(4)]
    with _on_device_of(vmem.device):
        _check(lib.exodus_synlif_backward(_ptr(inputGrad), *[_ptr(x) for x in per_row], _ptr(gradSpikes),
                                          _ptr(gradVmem), _ptr(gradIsyn), _ptr(vmem), _ptr(isyn),
                                          _ptr(vmemPostInitial), _ptr(isynInitial), _ptr(alphaMem), _ptr(alphaSyn),
                                          _ptr(membrSubtract), _ptr(theta), _ptr(thetaLow),
                                          int(bool(applyThetaLow)), int(maxNumSpikes), int(bool(decayEarly)),
                                          int(bool(normInput)), int(surrogateKind), float(surrP0), float(surrP1),
                                          n, t, _stream(vmem)), "exodus_synlif_backward")
    return (inputGrad, *per_row)


# ------------------------------------------------------------------------------------------
# layer-layout kernels: (batch, time, neurons) tensors, no transposition
# ------------------------------------------------------------------------------------------

# neurons per batch element the layer-layout entry points accept (they return invalid-value beyond)
LAYER_MAX_NEURONS = 1 << 25


_CHECKPOINT_INTERVAL = int(lib.exodus_layer_checkpoint_interval())


def checkpointInterval() -> int:
    return _CHECKPOINT_INTERVAL


def _btm(x: torch.Tensor, name: str, like: Optional[torch.Tensor] = None):
    _dev(x, name, like)
    if x.ndim != 3:
        raise RuntimeError(f"{name} must be 3-D (batch, time, neurons)")
    return x


def layerLifForward(input, vmemPostInitial, isynInitial, alphaMem, alphaSyn, membrSubtract, theta, thetaLow,
                    applyThetaLow: bool, maxNumSpikes: int, decayEarly: bool, normInput: bool,
                    wantCheckpoints: bool = True, wantRecords: bool = False, wantSpikeSum: bool = True,
                    outSpikes: Optional[torch.Tensor] = None, stateShape: Optional[tuple] = None,
                    wantPreReset: bool = False):
    """Returns dict(spikes, v_last, i_last, ckpt_v, ckpt_i, v_rec, i_rec, spike_sum); absent items are None.
    ``stateShape`` (product = batch*neurons) gives v_last / i_last that shape instead of a flat vector.
    ``wantRecords`` records potential (after the reset) and synaptic current of every step;
    ``wantPreReset`` records only the potential, before the reset (the surrogate function's argument)."""
    if wantRecords and wantPreReset:
        raise RuntimeError("wantRecords and wantPreReset exclude each other")
    _btm(input, "input")
    b, t, m = input.shape
    n = b * m
    syn = alphaSyn is not None
    rows = [("vmemPostInitial", vmemPostInitial), ("alphaMem", alphaMem), ("membrSubtract", membrSubtract),
            ("theta", theta)]
    if syn:
        rows += [("isynInitial", isynInitial), ("alphaSyn", alphaSyn)]
    for nm, x in rows:
        _rows(_dev(x, nm, input), nm, n)
    if applyThetaLow:
        _rows(_dev(thetaLow, "thetaLow", input), "thetaLow", n)
    else:
        thetaLow = None
    # big outputs go where hbm.enable() wants them (memory striped over the regions of HBM)
    spikes = hbm.empty_like(input) if outSpikes is None else outSpikes
    if spikes.shape != input.shape:
        raise RuntimeError("outSpikes must have the shape of input")
    _dev(spikes, "outSpikes", input)
    new = lambda *shape: (hbm.empty(shape, input) if len(shape) == 3
                          else torch.empty(shape, dtype=torch.float32, device=input.device))
    n_ck = (t + checkpointInterval() - 1) // checkpointInterval()
    state_shape = (n,) if stateShape is None else tuple(stateShape)
    if math.prod(state_shape) != n:
        raise RuntimeError(f"stateShape {state_shape} does not hold {n} neurons")
    res = dict(spikes=spikes, v_last=new(*state_shape), i_last=new(*state_shape) if syn else None,
               ckpt_v=new(b, n_ck, m) if wantCheckpoints else None,
               ckpt_i=new(b, n_ck, m) if (wantCheckpoints and syn) else None,
               v_rec=new(b, t, m) if (wantRecords or wantPreReset) else None,
               i_rec=new(b, t, m) if (wantRecords and syn) else None,
               spike_sum=torch.zeros((), dtype=torch.float64, device=input.device) if wantSpikeSum else None)
    if t == 0:                                   # nothing to integrate: the final states are the initial ones
        res["v_last"].copy_(vmemPostInitial.reshape(state_shape))
        if syn:
            res["i_last"].copy_(isynInitial.reshape(state_shape))
    with _on_device_of(input.device):
        _check(lib.exodus_layer_lif_forward(
            _ptr(spikes), _ptr(res["v_rec"]), _ptr(res["i_rec"]), _ptr(res["ckpt_v"]), _ptr(res["ckpt_i"]),
            _ptr(res["v_last"]), _ptr(res["i_last"]), _ptr(res["spike_sum"]), _ptr(input), _ptr(vmemPostInitial),
            _ptr(isynInitial) if syn else None, _ptr(alphaMem), _ptr(alphaSyn) if syn else None, _ptr(membrSubtract),
            _ptr(theta), _ptr(thetaLow), int(bool(applyThetaLow)), int(maxNumSpikes), int(bool(decayEarly)),
            int(bool(normInput)), int(bool(wantPreReset)), b, t, m, _stream(input)), "exodus_layer_lif_forward")
    return res


def backwardTimeSplit(mode: int = -1) -> int:
    """How ``layerLifBackward`` treats layers with few neurons and many steps (``exodus_layer_backward_time_split``):
    0 never splits the sequence over lanes, 1 (default) does for layers of up to 16 384 neurons, 2 whenever the kernel
    applies; -1 only asks.  Returns the mode that was set before."""
    return int(lib.exodus_layer_backward_time_split(int(mode)))


def scratchFloats() -> int:
    """Floats of checkpoint memory the library holds per GPU for ``layerLifBackward(..., ckptV=None)``."""
    return int(lib.exodus_layer_scratch_floats())


def layerLifBackward(gradSpikes, gradVLast, gradILast, input, ckptV, ckptI, vmemPostInitial, isynInitial, alphaMem,
                     alphaSyn, membrSubtract, theta, thetaLow, applyThetaLow: bool, maxNumSpikes: int,
                     decayEarly: bool, normInput: bool, surrogateKind: int, surrP0: float, surrP1: float,
                     gradInput: Optional[torch.Tensor] = None, surr: Optional[torch.Tensor] = None,
                     gradVRec: Optional[torch.Tensor] = None, gradIRec: Optional[torch.Tensor] = None,
                     wantAlphaMemGrad: bool = True, wantAlphaSynGrad: bool = True, wantVInitGrad: bool = True,
                     wantIInitGrad: bool = True, gradUniform: bool = False):
    """Returns (gradInput, alphaMemGrad, alphaSynGrad | None, vInitGrad, iInitGrad | None); a per-neuron
    gradient that is not wanted is neither computed nor allocated and comes back as None.
    ``gradUniform``: ``gradSpikes`` is a one-element tensor whose value is the gradient of every spike (the
    gradient of a sum of the output); the kernel then reads one tensor less.  Only with an in-kernel
    surrogate and without ``gradVRec`` / ``gradIRec``.
    ``surrogateKind == SURR_TENSOR`` takes the spike function's derivative from ``surr`` (batch, time, neurons).
    ``gradVRec`` / ``gradIRec`` (batch, time, neurons) are gradients on the forward's state records; one that is
    missing while the other is given counts as zero.
    ``ckptV is None`` calls ``exodus_layer_lif_backward_from_input``: the library rebuilds the checkpoints in its
    own fixed device array (``scratchFloats()``) and allocates nothing; concurrent calls on one GPU must not overlap."""
    _btm(input, "input")
    b, t, m = input.shape
    n = b * m
    syn = alphaSyn is not None
    if gradUniform:
        if _dev(gradSpikes, "gradSpikes", input).numel() != 1:
            raise RuntimeError("gradSpikes must hold one value when gradUniform is set")
        if surrogateKind == SURR_TENSOR or gradVRec is not None or gradIRec is not None:
            raise RuntimeError("gradUniform needs an in-kernel surrogate and no gradients on the state records")
    elif _btm(gradSpikes, "gradSpikes", input).shape != input.shape:
        raise RuntimeError("gradSpikes must have the shape of input")
    n_ck = (t + checkpointInterval() - 1) // checkpointInterval()
    from_input = ckptV is None
    if not from_input:
        for nm, x in (("ckptV", ckptV),) + ((("ckptI", ckptI),) if syn else ()):
            if _btm(x, nm, input).shape != (b, n_ck, m):
                raise RuntimeError(f"{nm} must have shape ({b}, {n_ck}, {m})")
    rows = [("vmemPostInitial", vmemPostInitial), ("alphaMem", alphaMem), ("membrSubtract", membrSubtract),
            ("theta", theta)]
    if syn:
        rows += [("isynInitial", isynInitial), ("alphaSyn", alphaSyn)]
    for nm, x in rows:
        _rows(_dev(x, nm, input), nm, n)
    for nm, x in (("gradVLast", gradVLast), ("gradILast", gradILast if syn else None)):
        if x is not None and _dev(x, nm, input).numel() != n:
            raise RuntimeError(f"{nm} must hold {n} values")
    if applyThetaLow:
        _rows(_dev(thetaLow, "thetaLow", input), "thetaLow", n)
    else:
        thetaLow = None
    if gradInput is None:
        gradInput = hbm.empty_like(input)
    elif _btm(gradInput, "gradInput", input).shape != input.shape:
        raise RuntimeError("gradInput must have the shape of input")
    if surrogateKind == SURR_TENSOR:
        if surr is None or _btm(surr, "surr", input).shape != input.shape:
            raise RuntimeError("surr must be given with the shape of input")
    else:
        surr = None
    if not syn:
        gradIRec = None
    if gradVRec is not None or gradIRec is not None:
        if gradVRec is None:
            gradVRec = torch.zeros_like(input)
        if syn and gradIRec is None:
            gradIRec = torch.zeros_like(input)
        for nm, x in (("gradVRec", gradVRec), ("gradIRec", gradIRec)):
            if x is not None and _btm(x, nm, input).shape != input.shape:
                raise RuntimeError(f"{nm} must have the shape of input")
    # the kernel writes every neuron's entry of each vector it is given -- unless there is no step to
    # walk: then nothing is launched, the decay factors have no influence and a gradient on a final
    # state is the gradient of the initial state it equals
    # (the wanted vectors are rows of one allocation)
    wanted = [bool(wantAlphaMemGrad), bool(wantVInitGrad), bool(syn and wantAlphaSynGrad), bool(syn and wantIInitGrad)]
    block = (torch.zeros if t == 0 else torch.empty)((sum(wanted), n), dtype=torch.float32, device=input.device)
    taken = iter(block.unbind(0))
    am_g, v0_g, as_g, i0_g = (next(taken) if w else None for w in wanted)
    if t == 0:
        if v0_g is not None and gradVLast is not None:
            v0_g.copy_(gradVLast.reshape(-1))
        if i0_g is not None and gradILast is not None:
            i0_g.copy_(gradILast.reshape(-1))
    head = (_ptr(gradInput), _ptr(am_g), _ptr(as_g), _ptr(v0_g), _ptr(i0_g), _ptr(gradSpikes), _ptr(gradVLast),
            _ptr(gradILast) if syn else None, _ptr(input))
    tail = (_ptr(vmemPostInitial), _ptr(isynInitial) if syn else None, _ptr(alphaMem), _ptr(alphaSyn) if syn else None,
            _ptr(membrSubtract), _ptr(theta), _ptr(thetaLow), int(bool(applyThetaLow)), int(maxNumSpikes),
            int(bool(decayEarly)), int(bool(normInput)), int(surrogateKind), float(surrP0), float(surrP1), _ptr(surr),
            _ptr(gradVRec), _ptr(gradIRec), int(bool(gradUniform)), b, t, m, _stream(input))
    with _on_device_of(input.device):
        if from_input:
            _check(lib.exodus_layer_lif_backward_from_input(*head, *tail), "exodus_layer_lif_backward_from_input")
        else:
            _check(lib.exodus_layer_lif_backward(*head, _ptr(ckptV), _ptr(ckptI) if syn else None, *tail),
                   "exodus_layer_lif_backward")
    return gradInput, am_g, as_g, v0_g, i0_g


def layerLeakyForward(input, vmemInitial, alpha, decayEarly: bool, normInput: bool,
                      stateShape: Optional[tuple] = None, wantSum: bool = False):
    """Leaky-integrator layer on (batch, time, neurons): returns (out, v_last), or with ``wantSum``
    (out, v_last, out_sum) where out_sum is a float64 scalar holding the sum of all outputs."""
    _btm(input, "input")
    b, t, m = input.shape
    n = b * m
    _rows(_dev(vmemInitial, "vmemInitial", input), "vmemInitial", n)
    _rows(_dev(alpha, "alpha", input), "alpha", n)
    state_shape = (n,) if stateShape is None else tuple(stateShape)
    if math.prod(state_shape) != n:
        raise RuntimeError(f"stateShape {state_shape} does not hold {n} neurons")
    out = hbm.empty_like(input)
    v_last = torch.empty(state_shape, dtype=torch.float32, device=input.device)
    out_sum = torch.zeros((), dtype=torch.float64, device=input.device) if wantSum else None
    if t == 0:
        v_last.copy_(vmemInitial.reshape(state_shape))
    with _on_device_of(input.device):
        _check(lib.exodus_layer_leaky_forward(_ptr(out), _ptr(v_last), _ptr(out_sum), _ptr(input), _ptr(vmemInitial),
                                              _ptr(alpha), int(bool(decayEarly)), int(bool(normInput)), b, t, m,
                                              _stream(input)), "exodus_layer_leaky_forward")
    return (out, v_last, out_sum) if wantSum else (out, v_last)


def layerLeakyBackward(gradOut, gradVLast, out, input, vmemInitial, alpha, decayEarly: bool, normInput: bool,
                       needAlphaGrad: bool, shape: Optional[tuple] = None):
    """Returns (gradInput, alphaGrad | None, vInitGrad).  With ``shape`` = (batch, time, neurons), ``gradOut`` is a
    one-element tensor whose value is the gradient of every output (the gradient of a sum)."""
    uniform = shape is not None
    if uniform:
        if _dev(gradOut, "gradOut").numel() != 1:
            raise RuntimeError("gradOut must hold one value when shape is given")
        b, t, m = (int(v) for v in shape)
    else:
        _btm(gradOut, "gradOut")
        b, t, m = gradOut.shape
    n = b * m
    _rows(_dev(alpha, "alpha", gradOut), "alpha", n)
    if gradVLast is not None and _dev(gradVLast, "gradVLast", gradOut).numel() != n:
        raise RuntimeError(f"gradVLast must hold {n} values")
    need_x = needAlphaGrad and (decayEarly or normInput)
    if needAlphaGrad:
        if tuple(_btm(out, "out", gradOut).shape) != (b, t, m):
            raise RuntimeError("out must have the shape of gradOut")
        _rows(_dev(vmemInitial, "vmemInitial", gradOut), "vmemInitial", n)
    if need_x and tuple(_btm(input, "input", gradOut).shape) != (b, t, m):
        raise RuntimeError("input must have the shape of gradOut")
    grad_input = hbm.empty((b, t, m), gradOut)
    block = torch.zeros((2 if needAlphaGrad else 1, n), dtype=torch.float32, device=gradOut.device)
    v_init_grad = block[0]
    alpha_grad = block[1] if needAlphaGrad else None
    if t == 0 and gradVLast is not None:
        v_init_grad.copy_(gradVLast.reshape(-1))
    with _on_device_of(gradOut.device):
        _check(lib.exodus_layer_leaky_backward(
            _ptr(grad_input), _ptr(alpha_grad), _ptr(v_init_grad), _ptr(gradOut), _ptr(gradVLast),
            _ptr(out) if needAlphaGrad else None, _ptr(input) if need_x else None,
            _ptr(vmemInitial) if needAlphaGrad else None, _ptr(alpha), int(bool(decayEarly)), int(bool(normInput)),
            int(uniform), b, t, m, _stream(gradOut)), "exodus_layer_leaky_backward")
    return grad_input, alpha_grad, v_init_grad
