"""Helpers shared by the parity tests (CPU-side; importing this never touches the GPU)."""
import torch

RTOL, ATOL = 1e-4, 1e-5          # fp32 tolerance for v_mem and gradients


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rel_err(got: torch.Tensor, want: torch.Tensor, rtol=RTOL, atol=ATOL) -> float:
    """max |got-want| / (atol + rtol |want|); <= 1 means within tolerance."""
    got = got.detach().cpu().double(); want = want.detach().cpu().double()
    if got.numel() == 0:
        return 0.0
    return ((got - want).abs() / (atol + rtol * want.abs())).max().item()


def assert_close(got, want, what, rtol=RTOL, atol=ATOL):
    e = rel_err(got, want, rtol, atol)
    assert e <= 1.0, f"{what}: error is {e:.3g} x tolerance (rtol={rtol}, atol={atol})"


def assert_close_rowscaled(got, want, what, rtol=RTOL, atol=ATOL):
    """|got - want| <= atol + rtol * max_t |want[row, :]|.

    For recurrences whose per-step factor exceeds 1 in magnitude (strong surrogate gradients) the
    rounding noise of a row's largest values reaches its small ones, so the error is judged against
    the magnitude that flows through the row rather than element by element."""
    got = got.detach().cpu().double(); want = want.detach().cpu().double()
    scale = want.abs().amax(dim=1, keepdim=True) if want.ndim == 2 else want.abs()
    e = ((got - want).abs() / (atol + rtol * scale)).max().item()
    assert e <= 1.0, f"{what}: error is {e:.3g} x row-scaled tolerance (rtol={rtol}, atol={atol})"


def spike_tie_report(s_got, s_want, v_want, theta, ulps=4):
    """Compare spike rasters row by row.

    A row may differ only if, at its FIRST differing step, the reference potential sits within
    `ulps` float32 ulps of an integer multiple of the threshold (an exact-threshold tie: one
    rounding decides the count, and everything after that step legitimately diverges).
    Returns (fraction of rows that differ through a tie, number of rows that differ otherwise).
    """
    s_got = s_got.detach().cpu(); s_want = s_want.detach().cpu(); v_want = v_want.detach().cpu()
    theta = theta.detach().cpu().reshape(-1, 1).expand_as(v_want)
    diff = s_got != s_want
    rows = diff.any(1).nonzero().flatten()
    ties = bad = 0
    for r in rows.tolist():
        t = int(diff[r].nonzero()[0])
        v, th = v_want[r, t].double(), theta[r, t].double()
        k = torch.round(v / th)
        eps = torch.finfo(torch.float32).eps * max(abs(v.item()), th.item())
        if abs((v - k * th).item()) <= ulps * eps:
            ties += 1
        else:
            bad += 1
    n = max(1, s_want.shape[0])
    return ties / n, bad


def lif_case(seed, n, t, *, lo=True, scale=0.5, shift=0.2):
    """Random per-row parameters for the spiking kernels."""
    g = gen(seed)
    d = dict(
        x=torch.randn(n, t, generator=g) * scale + shift,
        alpha=torch.rand(n, generator=g),
        v0=torch.randn(n, generator=g) * 0.3,
        theta=0.5 + torch.rand(n, generator=g),
        c=0.3 + 0.5 * torch.rand(n, generator=g),
        lo=(-0.2 - 0.4 * torch.rand(n, generator=g)) if lo else None,
        go=torch.randn(n, t, generator=g),
        gv=torch.randn(n, t, generator=g),
    )
    return d
