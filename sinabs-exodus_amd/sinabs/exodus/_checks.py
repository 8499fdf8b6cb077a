"""Argument checks shared by the autograd Functions.  Messages are those of the reference
(reference sinabs/exodus/spike.py:163-191, leaky.py:30-41) so that callers and tests that match on
them keep working."""
import torch


def check_rows_by_time(name: str, x: torch.Tensor) -> None:
    """``x`` must be a contiguous (N, Time) matrix."""
    if x.ndim != 2:
        raise ValueError(f"'{name}' must be 2D, (N, Time)")
    if not x.is_contiguous():
        raise ValueError(f"'{name}' has to be contiguous.")


def check_per_row(**named) -> None:
    """Every given tensor must be a contiguous (N,) vector; ``None`` entries are skipped."""
    for name, x in named.items():
        if x is None:
            continue
        if x.ndim != 1:
            raise ValueError(f"'{name}' must be 1D, (N,)")
        if not x.is_contiguous():
            raise ValueError(f"'{name}' has to be contiguous.")
