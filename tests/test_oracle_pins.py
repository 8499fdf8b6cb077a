"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each check is chosen so that a plausible mistake in the oracle (dropped term, wrong sign or
index, missing gate) fails it: the reference's own known answers (Gradient_analysis.ipynb
cells 2/4/6, tests/test_exp_leak.py:53-75), closed forms, brute force in float64, finite
differences and torch-autograd back-propagation through time.  Runs on the CPU.
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import exodus_ref as ref
from oracle import sinabs_cpu as sc


def f32(x):
    return torch.as_tensor(np.asarray(x), dtype=torch.float32).contiguous()


@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "notebook_kat.json")) as f:
        return json.load(f)


# ------------------------------------------------------------------ leaky forward
def leaky_closed_form(x, v0, a):
    """out_t = a^(t+1) v0 + sum_{k<=t} a^(t-k) x_k, in float64."""
    x = x.double().numpy(); v0 = v0.double().numpy(); a = a.double().numpy()
    n, t = x.shape
    out = np.zeros((n, t))
    for i in range(t):
        k = np.arange(i + 1)
        out[:, i] = a ** (i + 1) * v0 + (a[:, None] ** (i - k)[None, :] * x[:, : i + 1]).sum(1)
    return out


def test_leaky_forward_closed_form():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 33, generator=g); v0 = torch.randn(7, generator=g); a = torch.rand(7, generator=g)
    out = ref.leaky_forward(x, v0, a)
    np.testing.assert_allclose(out.numpy(), leaky_closed_form(x, v0, a), rtol=2e-5, atol=2e-6)


def test_leaky_forward_alpha_one_is_cumsum():
    g = torch.Generator().manual_seed(1)
    x = torch.randint(-8, 9, (5, 40), generator=g).float() / 16  # exactly representable sums
    v0 = torch.tensor([0.0, 0.5, -1.25, 2.0, 0.0625])
    out = ref.leaky_forward(x, v0, torch.ones(5))
    assert torch.equal(out, v0[:, None] + torch.cumsum(x, 1))


def test_leaky_forward_single_pulse_decay():
    # structure of reference tests/test_exp_leak.py:53-75: a pulse at t=0 decays as alpha^t
    alpha = torch.exp(-1 / torch.tensor(30.0))
    x = torch.zeros(3, 100); x[:, 0] = 1.0
    out = ref.leaky_forward(x, torch.zeros(3), alpha.expand(3).contiguous())
    assert torch.allclose(out[:, 0], torch.tensor(1.0))
    assert torch.isclose(out[:, -1], alpha ** 99, atol=1e-8).all()


# ------------------------------------------------------------------ leaky backward
def test_leaky_backward_is_transpose_of_forward():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 25, generator=g); go = torch.randn(6, 25, generator=g); a = torch.rand(6, generator=g)
    z = torch.zeros(6)
    lhs = (go.double() * ref.leaky_forward(x, z, a).double()).sum(1)
    rhs = (ref.leaky_backward(go, a).double() * x.double()).sum(1)
    np.testing.assert_allclose(lhs.numpy(), rhs.numpy(), rtol=1e-5, atol=1e-5)


def test_leaky_backward_flip_identity_and_closed_form():
    g = torch.Generator().manual_seed(3)
    go = torch.randn(4, 19, generator=g); a = torch.rand(4, generator=g)
    gi = ref.leaky_backward(go, a)
    flipped = ref.leaky_forward(go.flip(1).contiguous(), torch.zeros(4), a).flip(1)
    assert torch.equal(gi, flipped)
    # gi_t = sum_{j>=t} a^(j-t) go_j
    t = go.shape[1]
    want = np.zeros((4, t))
    for i in range(t):
        j = np.arange(i, t)
        want[:, i] = (a.double().numpy()[:, None] ** (j - i)[None, :] * go.double().numpy()[:, i:]).sum(1)
    np.testing.assert_allclose(gi.numpy(), want, rtol=2e-5, atol=2e-6)


def test_leaky_backward_alpha_finite_differences():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 30, generator=g); v0 = torch.randn(5, generator=g)
    a = 0.2 + 0.7 * torch.rand(5, generator=g); go = torch.randn(5, 30, generator=g)
    out = ref.leaky_forward(x, v0, a)
    ga = ref.leaky_backward_alpha(go, out, v0, a)
    h = 1e-6
    lp = (go.double().numpy() * leaky_closed_form(x, v0, a.double() + h)).sum(1)
    lm = (go.double().numpy() * leaky_closed_form(x, v0, a.double() - h)).sum(1)
    np.testing.assert_allclose(ga.numpy(), (lp - lm) / (2 * h), rtol=2e-4, atol=1e-4)
    # identity used by the fused kernels: grad_alpha = sum_t gi_t * out_{t-1}, out_{-1} = v_init
    gi = ref.leaky_backward(go, a).double()
    prev = torch.cat([v0[:, None], out[:, :-1]], 1).double()
    np.testing.assert_allclose(ga.numpy(), (gi * prev).sum(1).numpy(), rtol=2e-5, atol=2e-5)


# ------------------------------------------------------------------ spiking forward
def test_lif_forward_notebook_known_answers(kat):
    x = f32([kat["input"]])
    th = f32([kat["threshold"]]); a = f32([kat["alpha"]])
    for case in kat["cases"]:
        c = f32([case["membrane_subtract"]])
        s, v = ref.lif_forward(x, torch.zeros(1), a, c, th, None, False, -1)
        if case["spikes"] is not None:
            assert s[0].tolist() == case["spikes"], case["name"]
        np.testing.assert_allclose(v[0].numpy(), case["v_mem_pre_reset"], atol=case["v_mem_abs_tol"])


def test_iaf_forward_is_floor_of_cumsum():
    # alpha=1, subtract=threshold, no clamp, x>=0: cumulative spike count = floor(cumsum(x)/theta)
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 40, (9, 64), generator=g).float() / 16
    th = torch.full((9,), 1.0)
    s, v = ref.lif_forward(x, torch.zeros(9), torch.ones(9), th, th, None, False, -1)
    assert torch.equal(torch.cumsum(s, 1), torch.floor(torch.cumsum(x, 1)))
    assert torch.equal(v - s, torch.cumsum(x, 1) - torch.cumsum(s, 1))  # post-reset potential in [0,1)
    assert ((v - s) >= 0).all() and ((v - s) < 1).all()


def test_lif_forward_cap_clamp_and_threshold_edge():
    th = f32([1.0, 1.0, 1.0, 0.5])
    x = f32([[3.5, 0, 0, 0], [3.5, 0, 0, 0], [-5, 0.5, 1.0, 0], [1.0, 0.25, 0.25, -9]])
    a = f32([1.0, 1.0, 0.5, 1.0]); lo = f32([-1, -1, -1, -2])
    # no cap: 3 spikes, then the remaining 0.5 stays below threshold
    s, v = ref.lif_forward(x[:1].contiguous(), torch.zeros(1), a[:1], th[:1], th[:1], None, False, -1)
    assert s[0].tolist() == [3, 0, 0, 0] and v[0].tolist() == [3.5, 0.5, 0.5, 0.5]
    # cap 1: one spike per step until the charge is used up
    s, v = ref.lif_forward(x[1:2].contiguous(), torch.zeros(1), a[1:2], th[1:2], th[1:2], None, False, 1)
    assert s[0].tolist() == [1, 1, 1, 0] and v[0].tolist() == [3.5, 2.5, 1.5, 0.5]
    # clamp at -1 then decay 0.5: v = -1, -0.5+0.5=0, 0+1=1 -> fires at exactly theta (>=)
    s, v = ref.lif_forward(x[2:3].contiguous(), torch.zeros(1), a[2:3], th[2:3], th[2:3], lo[2:3], True, -1)
    assert v[0].tolist() == [-1.0, 0.0, 1.0, 0.0] and s[0].tolist() == [0, 0, 1, 0]
    # threshold 0.5, v=1.0 -> 2 spikes; negative potential never fires and is clamped at -2
    s, v = ref.lif_forward(x[3:4].contiguous(), torch.zeros(1), a[3:4], th[3:4], th[3:4], lo[3:4], True, -1)
    assert s[0].tolist() == [2, 0, 1, 0] and v[0].tolist() == [1.0, 0.25, 0.5, -2.0]


def test_lif_forward_nonzero_initial_state_and_subtract():
    # v_init is post-reset: first step is alpha*v_init + x
    s, v = ref.lif_forward(f32([[0.25, 0.0]]), f32([0.5]), f32([0.5]), f32([0.25]), f32([0.5]), None, False, -1)
    assert v[0].tolist() == [0.5, (0.5 - 0.25) * 0.5] and s[0].tolist() == [1, 0]


# ------------------------------------------------------------------ spiking backward
def test_lif_backward_notebook_known_answers(kat):
    th = kat["threshold"]
    x = f32([kat["input"]])
    for case in kat["cases"]:
        c = case["membrane_subtract"]
        surr = torch.full((1, 5), 1.0 / th)
        go = torch.zeros(1, 5); go[0, -1] = 1.0           # d a_5 / d I
        g = (surr * go).contiguous()
        gi = ref.lif_backward(surr, g, torch.ones(1, 5), f32([1.0]), f32([1.0 * c]))
        want = np.asarray(case["grad_of_last_spike_wrt_input"])
        np.testing.assert_allclose(gi[0].numpy(), want, rtol=case["grad_rel_tol"], atol=1e-7)
        # the same through the Function-level glue with the Heaviside surrogate of cell 1
        s, v = ref.lif_forward(x, torch.zeros(1), f32([1.0]), f32([c]), f32([th]), None, False, -1)
        gi2, _, ginit = ref.integrate_and_fire_backward(go, None, v, s, torch.zeros(1), f32([1.0]), f32([c]),
                                                        f32([th]), None, ref.Heaviside(window=th), False)
        np.testing.assert_allclose(gi2[0].numpy(), want, rtol=case["grad_rel_tol"], atol=1e-7)
        np.testing.assert_allclose(ginit.numpy(), want[:1], rtol=case["grad_rel_tol"], atol=1e-7)


def _random_backward_case(seed, n=6, t=23, clip=True):
    g = torch.Generator().manual_seed(seed)
    surr = torch.rand(n, t, generator=g)
    gg = torch.randn(n, t, generator=g)
    nc = (torch.rand(n, t, generator=g) > 0.25).float() if clip else torch.ones(n, t)
    a = torch.rand(n, generator=g)
    c = 0.2 + torch.rand(n, generator=g)
    return surr, gg, nc, a, c


def test_lif_backward_matches_product_closed_form():
    # d a_T / d I_t of notebook cell 7, contracted with g:  brute force over all (i, j) in float64
    surr, g, nc, a, c = _random_backward_case(6)
    gi = ref.lif_backward(surr, g, nc, a, (a * c).contiguous())
    S, G, NC = surr.double().numpy(), g.double().numpy(), nc.double().numpy()
    A, C = a.double().numpy(), (a * c).double().numpy()
    n, t = S.shape
    want = np.zeros((n, t))
    for r in range(n):
        for i in range(t):
            for j in range(i, t):
                prod = NC[r, i]
                for k in range(i + 1, j + 1):
                    prod *= (A[r] - C[r] * S[r, k - 1]) * NC[r, k]
                want[r, i] += prod * G[r, j]
    np.testing.assert_allclose(gi.numpy(), want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("clip", [False, True])
def test_lif_backward_equals_linear_recurrence(clip):
    surr, g, nc, a, c = _random_backward_case(7, n=8, t=50, clip=clip)
    gi = ref.lif_backward(surr, g, nc, a, (a * c).contiguous())
    gi64, _, ginit64 = ref.lif_backward_recurrence_f64(surr, g, nc, a, c)
    np.testing.assert_allclose(gi.numpy(), gi64.numpy(), rtol=2e-5, atol=2e-6)


def _bptt(x, v0, a, c, th, lo, surrogate, cap, w_spk, w_v, clip_mode="max"):
    """Gradients of sum(w_spk*spikes + w_v*v_pre_reset) by autograd through the step loop."""
    x = x.clone().requires_grad_(True); v0 = v0.clone().requires_grad_(True); a = a.clone().requires_grad_(True)
    inp = x.t().unsqueeze(0)                                 # (1, T, n)
    out, state, rec = sc.lif_forward(inp, a, None, {"v_mem": v0.unsqueeze(0)}, th, c, surrogate, cap,
                                     lo, norm_input=False, clip_mode=clip_mode)
    loss = (out[0].t() * w_spk).sum() + (rec["v_mem"][0].t() * w_v).sum()
    loss.backward()
    return out[0].t().detach(), rec["v_mem"][0].t().detach(), x.grad, a.grad, v0.grad


@pytest.mark.parametrize("surrogate", [ref.Heaviside(0.4), ref.SingleExponential(), ref.PeriodicExponential()])
@pytest.mark.parametrize("use_lo,cap,v0_zero", [(False, None, True), (True, 2, True), (True, None, False),
                                                 (False, 1, False)])
def test_function_glue_matches_autograd_bptt(surrogate, use_lo, cap, v0_zero):
    g = torch.Generator().manual_seed(11)
    n, t = 12, 40
    x = torch.randn(n, t, generator=g) * 0.6 + 0.2
    a = 0.5 + 0.5 * torch.rand(n, generator=g)
    th = 0.5 + torch.rand(n, generator=g)
    c = 0.3 + torch.rand(n, generator=g) * 0.5
    lo = -0.3 * torch.ones(n) if use_lo else None
    # keep step 0 unclipped when v_init != 0, where the reference alpha-gradient is exact
    v0 = torch.zeros(n) if v0_zero else torch.rand(n, generator=g) * 0.4
    if not v0_zero:
        x[:, 0] = x[:, 0].abs()
    w_spk = torch.randn(n, t, generator=g); w_v = torch.randn(n, t, generator=g)

    s_b, v_b, gx_b, ga_b, gv0_b = _bptt(x, v0, a, c, th, lo, surrogate, cap, w_spk, w_v)
    s, v = ref.integrate_and_fire_forward(x, a, v0, th, c, lo, cap)
    assert torch.equal(s, s_b) and torch.equal(v, v_b)       # same operations in the same order
    gi, ga, ginit = ref.integrate_and_fire_backward(w_spk, w_v, v, s, v0, a, c, th, lo, surrogate, True)
    np.testing.assert_allclose(gi.numpy(), gx_b.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ginit.numpy(), gv0_b.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ga.numpy(), ga_b.numpy(), rtol=2e-4, atol=2e-5)
    # and the single-reverse-pass identities used by the fused kernel
    surr = surrogate(v, th.unsqueeze(1)); ncl = (v > lo.unsqueeze(1)).float() if use_lo else torch.ones_like(v)
    gg = surr * w_spk + w_v
    gi64, ga64, gin64 = ref.lif_backward_recurrence_f64(surr, gg, ncl, a, c, v - c.unsqueeze(1) * s, v0)
    np.testing.assert_allclose(gi64.numpy(), gx_b.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ga64.numpy(), ga_b.numpy(), rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(gin64.numpy(), gv0_b.numpy(), rtol=1e-4, atol=1e-5)


def test_alpha_gradient_initial_step_gate():
    """Step 0 clipped with v_init != 0: the exact derivative gates v_init by nc_0, the reference
    device code (cuda/lif_kernels.h:219-234) does not.  gate_initial=True must equal autograd."""
    n, t = 4, 12
    g = torch.Generator().manual_seed(13)
    x = torch.randn(n, t, generator=g) * 0.5 + 0.3
    x[:, 0] = -3.0                                            # forces a clip at step 0
    a = 0.6 + 0.3 * torch.rand(n, generator=g); th = torch.ones(n); c = th.clone()
    lo = -0.5 * torch.ones(n); v0 = 0.5 + torch.rand(n, generator=g)
    w = torch.randn(n, t, generator=g)
    sur = ref.SingleExponential()
    s_b, v_b, gx_b, ga_b, _ = _bptt(x, v0, a, c, th, lo, sur, None, w, torch.zeros(n, t))
    s, v = ref.integrate_and_fire_forward(x, a, v0, th, c, lo, None)
    assert (v[:, 0] == lo).all()
    _, ga_exact, _ = ref.integrate_and_fire_backward(w, None, v, s, v0, a, c, th, lo, sur, True, gate_initial=True)
    _, ga_quirk, _ = ref.integrate_and_fire_backward(w, None, v, s, v0, a, c, th, lo, sur, True, gate_initial=False)
    np.testing.assert_allclose(ga_exact.numpy(), ga_b.numpy(), rtol=2e-4, atol=2e-5)
    assert (ga_exact - ga_quirk).abs().max() > 1e-3           # the two forms really differ here


# ------------------------------------------------------------------ sinabs-style loop vs kernel restatement
@pytest.mark.parametrize("cap", [None, 1, 3])
def test_step_loop_and_kernel_restatement_agree_bitwise(cap):
    g = torch.Generator().manual_seed(17)
    b, t, m = 3, 60, 11
    x = torch.randn(b, t, m, generator=g) * 0.7 + 0.2
    a = torch.rand(m, generator=g); th = 0.5 + torch.rand(m, generator=g); lo = -0.4
    out, state, rec = sc.lif_forward(x, a, None, {"v_mem": torch.zeros(b, m)}, th, None, ref.Heaviside(),
                                     cap, lo, norm_input=False, clip_mode="max")
    rows = sc.bt_to_rows(x)
    ex = lambda p: p.expand(b, m).flatten().contiguous()
    s, v = ref.integrate_and_fire_forward(rows, ex(a), torch.zeros(b * m), ex(th), None,
                                          torch.full((b * m,), lo), cap)
    assert torch.equal(sc.rows_to_bt(s, b), out)
    assert torch.equal(sc.rows_to_bt(v, b), rec["v_mem"])
    # the relu formulation of the clamp differs only by rounding on unclipped steps
    out_r, _, rec_r = sc.lif_forward(x, a, None, {"v_mem": torch.zeros(b, m)}, th, None, ref.Heaviside(),
                                     cap, lo, norm_input=False, clip_mode="relu")
    clipped = rec["v_mem"] == lo
    assert torch.equal(rec_r["v_mem"][clipped], rec["v_mem"][clipped])


def test_leaky_step_loop_matches_kernel_restatement():
    g = torch.Generator().manual_seed(19)
    b, t, m = 2, 50, 8
    x = torch.randn(b, t, m, generator=g); a = torch.rand(m, generator=g); v0 = torch.randn(b, m, generator=g)
    out, state, _ = sc.lif_forward(x, a, None, {"v_mem": v0}, None, None, None, None, None, False, spiking=False)
    rows = ref.leaky_forward(sc.bt_to_rows(x), v0.flatten().contiguous(), a.expand(b, m).flatten().contiguous())
    assert torch.equal(sc.rows_to_bt(rows, b), out)


def test_surrogate_closed_values():
    th = torch.tensor([[1.0], [2.0]])
    v = torch.tensor([[1.0, 0.5, 2.5], [2.0, 1.0, 5.0]])
    se = ref.SingleExponential(grad_width=0.5, grad_scale=1.0)(v, th)
    want = 1.0 / (th * 0.5) * torch.exp(-(v - th).abs() / (th * 0.5))
    assert torch.allclose(se, want)
    assert torch.allclose(se[:, 0], torch.tensor([2.0, 1.0]))          # peak value scale/(theta*w) at v=theta
    hv = ref.Heaviside(window=0.5)(v, th)
    assert hv.tolist() == [[1.0, 1.0, 1.0], [0.5, 0.0, 0.5]]
    pe = ref.PeriodicExponential()(v, th)
    # peak 1/theta at v = theta and again one period later; same value half a period either side
    assert torch.allclose(pe[:, 0], torch.tensor([1.0, 0.5]))
    assert torch.allclose(ref.PeriodicExponential()(torch.tensor([[2.0]]), torch.tensor([[1.0]])), torch.tensor([[1.0]]))
    assert torch.allclose(ref.PeriodicExponential()(torch.tensor([[1.5]]), torch.tensor([[1.0]])),
                          ref.PeriodicExponential()(torch.tensor([[0.5]]), torch.tensor([[1.0]])))


# ------------------------------------------------------------------ experimental spike generation
def test_spike_forward_notebook_known_answer(kat):
    """The notebook's neuron (alpha = 1) seen from the other side: its potential without resets is
    cumsum(input); spike generation on that must give the notebook's spikes and potentials."""
    case = kat["cases"][0]
    u = f32([kat["input"]]).cumsum(1).contiguous()
    s = ref.spike_forward(u, 1.0, case["membrane_subtract"], kat["threshold"], 0.0, False, -1)
    assert s[0].tolist() == case["spikes"]
    np.testing.assert_allclose(u[0].numpy(), case["v_mem_pre_reset"], atol=case["v_mem_abs_tol"])


@pytest.mark.parametrize("use_lo,cap", [(False, -1), (True, -1), (True, 2), (False, 1)])
def test_spike_forward_equals_lif_forward_on_dyadic_grid(use_lo, cap):
    """alpha = 1/2, inputs on a 1/64 grid, few steps: every product and sum below is exact in
    float32, so "leaky integral, then spike generation" and the LIF recurrence must agree to the
    bit although they order the arithmetic differently.  A clamped step keeps its own value in the
    spike function (only later steps are raised), hence the max()."""
    g = torch.Generator().manual_seed(17 + cap)
    n, t, a, th, c, lo = 64, 9, 0.5, 1.0, 0.75, -0.5
    x = (torch.randint(-96, 192, (n, t), generator=g).float() / 64.0).contiguous()
    ones = torch.ones(n)
    u = ref.leaky_forward(x, torch.zeros(n), a * ones)
    s_exp = ref.spike_forward(u, a, c, th, lo, use_lo, cap)
    s_lif, v_lif = ref.lif_forward(x, torch.zeros(n), a * ones, c * ones, th * ones, lo * ones, use_lo, cap)
    assert s_lif.sum() > 50 and (not use_lo or (u < lo).any())
    assert torch.equal(s_exp, s_lif)
    assert torch.equal(torch.clamp(u, min=lo) if use_lo else u, v_lif)


def test_spike_backward_notebook_known_answers(kat):
    """alpha = 1, nothing clipped: the gradient with respect to the input current is the leaky
    adjoint (reverse cumulative sum) of the gradient with respect to the potential."""
    th = kat["threshold"]
    for case in kat["cases"]:
        surr = torch.full((1, 5), 1.0 / th)
        go = torch.zeros(1, 5); go[0, -1] = 1.0
        gu = ref.spike_backward(surr, go, torch.ones(1, 5), 1.0, case["membrane_subtract"])
        gi = ref.leaky_backward(gu, f32([1.0]))
        np.testing.assert_allclose(gi[0].numpy(), case["grad_of_last_spike_wrt_input"],
                                   rtol=case["grad_rel_tol"], atol=2e-7)


def test_spike_backward_alpha_one_equals_production_backward():
    surr, gg, _, _, _ = _random_backward_case(5, clip=False)
    surr = surr * 0.8
    n, t = surr.shape
    ones = torch.ones(n)
    gu = ref.spike_backward(surr, gg, torch.ones(n, t), 1.0, 0.7)
    got = ref.leaky_backward(gu, ones)
    want = ref.lif_backward(surr, (surr * gg).contiguous(), torch.ones(n, t), ones, 0.7 * ones)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("alpha", [1.0, 0.8])
def test_spike_backward_quadratic_sum_equals_reverse_recurrence(alpha):
    """Two different algorithms for the same vector (the only check for alpha != 1 and for
    clipped steps, where no known answer of the reference exists)."""
    surr, gg, nc, _, _ = _random_backward_case(8)
    c = 0.6
    got = ref.spike_backward(surr, gg, nc, alpha, c).double()
    y = (surr * nc).double(); go = gg.double()
    m = torch.zeros(surr.shape[0], dtype=torch.float64)
    want = torch.zeros_like(go)
    for i in range(surr.shape[1] - 1, -1, -1):
        want[:, i] = y[:, i] * go[:, i] - y[:, i] * c * m
        m = go[:, i] * y[:, i] + (alpha - c * y[:, i]) * m
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-4, atol=1e-5)


class _Surrogate(torch.autograd.Function):
    """spike count (value taken from `counts`) whose derivative with respect to the potential is `surr`"""

    @staticmethod
    def forward(ctx, u, counts, surr):
        ctx.save_for_backward(surr)
        return counts.clone()

    @staticmethod
    def backward(ctx, g):
        (surr,) = ctx.saved_tensors
        return g * surr, None, None


def _spike_function_autograd(v, alpha, c, theta, lo, use_lo, surr, as_backward_formula=False):
    """The experimental spike generation as a float64 torch step loop, differentiated by autograd, with
    ds/du := surr.  Returns (leaf v, spikes).

    as_backward_formula=False: what oracle_spike_forward computes (reference
    cuda/experimental_kernels.h:33-63): every spike lowers the following steps by alpha^j c count,
    j = 1, 2, ..., and a step below the lower bound raises them by alpha^j (lo - u).
    as_backward_formula=True: the model whose exact gradient the reference's backward formula is
    (cuda/experimental_kernels.h:118-140): the first following step loses c count undecayed (alpha^(j-1)),
    and the amount a clipped step adds to later steps is treated as a constant."""
    n, t = v.shape
    v = v.double().clone().requires_grad_(True)
    adj = torch.zeros(n, dtype=torch.float64)          # what earlier steps add to this one
    spikes = []
    for i in range(t):
        u = v[:, i] + adj
        counts = torch.where(u >= theta, torch.div(u, theta, rounding_mode="trunc"), torch.zeros_like(u)).detach()
        below = (u < lo) & (u < theta) if use_lo else torch.zeros_like(u, dtype=torch.bool)
        y = surr[:, i].double()
        s = _Surrogate.apply(u, counts, torch.where(below, torch.zeros_like(y), y) if as_backward_formula else y)
        spikes.append(s)
        d = -c * s
        if use_lo:
            lift = lo - u
            d = torch.where(below, lift.detach() if as_backward_formula else lift, d)
        adj = alpha * adj + d if as_backward_formula else alpha * (adj + d)
    return v, torch.stack(spikes, 1)


@pytest.mark.parametrize("use_lo", [False, True])
@pytest.mark.parametrize("alpha", [1.0, 0.9, 0.6])
def test_spike_backward_is_the_exact_gradient_of_a_stated_model(alpha, use_lo):
    """Pins oracle_spike_backward for alpha != 1 and for clipped steps against autograd through an
    independent step loop.  The reference's sum (cuda/experimental_kernels.h:118-140) has the factors
    (alpha - c y_k) where its own forward pass (:33-63, first affected step already decayed) would give
    alpha (1 - c y_k): term by term it is the exact gradient of a forward pass in which a spike reaches the
    next step undecayed and a clipped step's contribution to later steps counts as a constant.  That is
    checked here; the distance to the exact gradient of the actual forward pass is printed (zero at
    alpha = 1 without clipped steps)."""
    g = torch.Generator().manual_seed(31)
    n, t, c, theta, lo = 48, 40, 0.6, 1.0, -0.3
    x = torch.randn(n, t, generator=g) * 0.6 + 0.25
    v = ref.leaky_forward(x.contiguous(), torch.zeros(n), alpha * torch.ones(n))
    surr = (torch.rand(n, t, generator=g) * 1.2).contiguous()          # the backward takes them as given
    go = torch.randn(n, t, generator=g).contiguous()
    # the actual forward pass: same spike trains as the oracle, so the same function
    leaf, s = _spike_function_autograd(v, alpha, c, theta, lo, use_lo, surr)
    u = v.clone()
    s_oracle = ref.spike_forward(u, alpha, c, theta, lo, use_lo, -1)
    assert s.sum() > 50 and torch.equal(s.detach().float(), s_oracle)
    (s * go.double()).sum().backward()
    exact = leaf.grad
    nc = (u > lo).float().contiguous() if use_lo else torch.ones(n, t)   # what reference spike.py:88-92 hands over
    assert not use_lo or 0 < (nc == 0).sum() < nc.numel() // 2
    got = ref.spike_backward(surr, go, nc, alpha, c).double()
    # the model of the backward formula, run on potentials that clip exactly where `nc` says
    leaf2, s2 = _spike_function_autograd(u.double() if use_lo else v, alpha, c, theta, lo, False, surr * nc, True)
    (s2 * go.double()).sum().backward()
    np.testing.assert_allclose(got.numpy(), leaf2.grad.numpy(), rtol=1e-4, atol=1e-5)
    dev = (got - exact).abs().max().item()
    print(f"alpha={alpha} lower bound={use_lo}: largest |reference formula - exact gradient of the forward pass| = "
          f"{dev:.3g} (largest gradient {exact.abs().max().item():.3g})")
    if alpha == 1.0 and not use_lo:
        np.testing.assert_allclose(got.numpy(), exact.numpy(), rtol=1e-4, atol=1e-5)
    else:
        assert dev > 1e-3                                               # not a rounding matter
