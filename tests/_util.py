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


# Assertions judged with a tolerance other than the stated one (sums of many products get an absolute
# tolerance scaled with the number of terms) leave their worst error in units of the STATED tolerance
# here; tests/conftest.py prints the table at the end of the run.  what -> (error in stated units, error
# in the units the assertion used, rtol used, atol used)
SCALED_TOLERANCE_REPORT = {}


def note_scaled(what, got, want, rtol, atol, used=None):
    """Record the worst error of (got, want) in units of rtol 1e-4 / atol 1e-5."""
    stated = rel_err(got, want, RTOL, ATOL)
    used = rel_err(got, want, rtol, atol) if used is None else used
    old = SCALED_TOLERANCE_REPORT.get(what)
    if old is None or stated > old[0]:
        SCALED_TOLERANCE_REPORT[what] = (stated, used, rtol, atol)


def assert_close(got, want, what, rtol=RTOL, atol=ATOL):
    e = rel_err(got, want, rtol, atol)
    if rtol != RTOL or atol != ATOL:
        note_scaled(what, got, want, rtol, atol, e)
    assert e <= 1.0, (f"{what}: error is {e:.3g} x tolerance (rtol={rtol}, atol={atol}); "
                      f"{rel_err(got, want, RTOL, ATOL):.3g} x the stated tolerance (rtol={RTOL}, atol={ATOL})")


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


def synaptic_layer_oracle(ref, x, go, am, asn, v0, i0, th, c, lo, cap, decay_early, norm_input, surrogate,
                          g_v_last=None, g_i_last=None):
    """Synapse -> membrane on (rows, time) matrices, composed from the oracle's restatements of the
    reference kernels exactly as the reference layer composes its Functions, with the elementwise glue
    and its chain rule written out (reference sinabs/exodus/layers/lif.py:185-254):
    input scaling (decay_early), LeakyIntegrator, input normalisation (norm_input), IntegrateAndFire.
    ``asn is None`` means a layer without synaptic current.  ``g_v_last`` / ``g_i_last`` are gradients
    arriving at the final states (post-reset potential, synaptic current).  Returns a dict with the
    forward results and every gradient."""
    syn = asn is not None
    if syn:
        xin = (x * asn[:, None]).contiguous() if decay_early else x.contiguous()
        i = ref.leaky_forward(xin, i0, asn)
    else:
        i = x.contiguous()
    u = ((1.0 - am)[:, None] * i).contiguous() if norm_input else i
    s, v = ref.integrate_and_fire_forward(u, am, v0, th, c, lo, None if cap < 0 else cap)
    out = dict(spikes=s, v_mem=v, i_syn=i, v_last=(v - c[:, None] * s)[:, -1], i_last=i[:, -1])
    if go is None:
        return out
    go = go.clone()
    g_vm = None
    if g_v_last is not None:            # final potential = v - c * spikes at the last step
        g_vm = torch.zeros_like(v)
        g_vm[:, -1] = g_v_last
        go[:, -1] -= c * g_v_last
    g_u, g_am, g_v0 = ref.integrate_and_fire_backward(go.contiguous(), g_vm, v, s, v0, am, c, th, lo, surrogate, True,
                                                      gate_initial=True)
    g_i = (1.0 - am)[:, None] * g_u if norm_input else g_u.clone()
    if norm_input:
        g_am = g_am - (g_u.double() * i.double()).sum(1).float()
    out.update(g_alpha_mem=g_am, g_v_init=g_v0)
    if not syn:
        out["g_x"] = g_i
        return out
    if g_i_last is not None:
        g_i = g_i.clone()
        g_i[:, -1] += g_i_last
    g_xin, g_as, g_i0 = ref.leaky_integrator_backward(g_i.contiguous(), i, i0, asn, True)
    if decay_early:
        g_as = g_as + (g_xin.double() * x.double()).sum(1).float()
        out["g_x"] = g_xin * asn[:, None]
    else:
        out["g_x"] = g_xin
    out.update(g_alpha_syn=g_as, g_i_init=g_i0)
    return out


def worst(got, want, rtol=RTOL, atol=ATOL) -> str:
    """The largest error in units of the stated tolerance, for printing next to an assertion that uses a
    scaled one."""
    return f"{rel_err(got, want, rtol, atol):.3g} x (rtol {rtol:g}, atol {atol:g})"
