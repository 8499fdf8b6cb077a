"""Value checks on device-resident parameters.

The reference Functions test ``0 <= alpha <= 1`` and ``threshold > min_v_mem`` with ``.any()`` on
device tensors (reference sinabs/exodus/spike.py:183-191), which makes the host wait for the device
on every forward call.  Three modes, selected with ``set_mode``:

``"sync"`` (default)   the reference's behaviour: one device-to-host transfer per call, the
                        ``ValueError`` is raised before any kernel is launched;
``"deferred"``          the flags are copied to pinned host memory without waiting; a violation is
                        raised by a later call into this module (or by ``flush()``), so the host can
                        keep queueing work;
``"off"``               no checks.

While the current stream is capturing a HIP graph no check runs in any mode: the capture cannot wait
for the device, and a replay has no host code that could raise.
"""
from typing import List, Optional, Sequence

import torch

_MODE = "sync"
_ALPHA_MSG = "'alpha' must be between 0 and 1."
_THRESHOLD_MSG = "`threshold` must be greater than `min_v_mem`."
_pending: List[tuple] = []          # (event, pinned flags, messages)


def set_mode(mode: str) -> None:
    global _MODE
    if mode not in ("sync", "deferred", "off"):
        raise ValueError("mode must be 'sync', 'deferred' or 'off'")
    flush()
    _MODE = mode


def get_mode() -> str:
    return _MODE


def _raise_if_flagged(flags: Sequence, messages: Sequence[str]) -> None:
    for flag, msg in zip(flags, messages):
        if flag:
            raise ValueError(msg)


def _poll(wait: bool) -> None:
    while _pending:
        event, host_flags, messages = _pending[0]
        if not wait and not event.query():
            return
        if wait:
            event.synchronize()
        _pending.pop(0)
        _raise_if_flagged(host_flags.tolist(), messages)


def flush() -> None:
    """Wait for all deferred checks and raise the first violation found."""
    _poll(wait=True)


def check_parameters(alphas: Sequence[torch.Tensor], threshold: Optional[torch.Tensor] = None,
                     min_v_mem: Optional[torch.Tensor] = None) -> None:
    """``alphas``: decay factors that must lie in [0, 1]; ``threshold`` must exceed ``min_v_mem``."""
    if _MODE == "off":
        return
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        return          # a graph under capture can neither wait for the device nor raise on replay
    if _MODE == "deferred":
        _poll(wait=False)
    flags = [((a < 0) | (a > 1)).any() for a in alphas]
    messages = [_ALPHA_MSG] * len(flags)
    if min_v_mem is not None:
        flags.append((threshold <= min_v_mem).any())
        messages.append(_THRESHOLD_MSG)
    if not flags:
        return
    stacked = torch.stack(flags)
    if _MODE == "sync" or not stacked.is_cuda:
        _raise_if_flagged(stacked.tolist(), messages)
        return
    host = torch.empty(stacked.shape, dtype=stacked.dtype, pin_memory=True)
    host.copy_(stacked, non_blocking=True)
    event = torch.cuda.Event()
    event.record(torch.cuda.current_stream(stacked.device))
    _pending.append((event, host, messages))
