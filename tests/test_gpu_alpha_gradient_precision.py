"""Gradients of the decay factors are sums of T products.  Elsewhere they are compared with the fp32 CPU oracle under
an absolute tolerance scaled by sqrt(T) (and reported in units of the stated rtol 1e-4 / atol 1e-5 at the end of the run):
two fp32 summations of 2000 terms in different orders differ by more than atol 1e-5 without either being wrong.

Here the question is settled against a float64 evaluation of the same sums (same fp32 forward values, recurrences and
sums in double).  For the spiking configuration the kernels -- fp32 fused multiply-adds over 32 steps, folded into a
double total -- must lie within the STATED tolerance of the float64 value, and at least as close to it as the oracle's
plain fp32 accumulation does.  For the leaky integrator under a gradient of ones the terms are of order 100 and largely
cancel (sums of 1000 terms between -6e4 and 6e4, some near zero), and the adjoint itself is an fp32 recurrence of 1000
steps in kernel and oracle alike: no fp32 evaluation can promise more than a few units in the last place of the summed
magnitudes, so there the allowance is the stated tolerance plus 2^-22 (four fp32 ulps) of sum_t |term_t|."""
import math

import pytest
import torch

from _util import ATOL, RTOL, gen, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip
    from oracle import exodus_ref as ref
    return _hip, ref


def judge(what, got, oracle32, exact, magnitude=None):
    """got (kernel), oracle32 (fp32 CPU oracle) and exact (float64), all on the CPU.  ``magnitude`` = sum of the
    absolute values of the summed terms per element (float64), where cancellation makes it the relevant scale."""
    got, oracle32 = got.detach().cpu().double(), oracle32.detach().cpu().double()
    ek, eo = rel_err(got, exact), rel_err(oracle32, exact)
    print(f"\n{what}: kernel {ek:.3g} x, fp32 oracle {eo:.3g} x the stated tolerance away from the float64 value; "
          f"kernel against oracle {rel_err(got, oracle32):.3g} x")
    if magnitude is None:
        assert ek <= 1.0, f"{what}: the kernel is {ek:.3g} x the stated tolerance (rtol {RTOL}, atol {ATOL}) from the float64 value"
        worst_k, worst_o = (got - exact).abs().max().item(), (oracle32 - exact).abs().max().item()
        assert worst_k <= worst_o + ATOL, f"{what}: kernel error {worst_k:.3g} exceeds the fp32 oracle's {worst_o:.3g}"
        return
    allowed = ATOL + RTOL * exact.abs() + magnitude * 2.0 ** -22
    for name, value in (("kernel", got), ("fp32 oracle", oracle32)):
        worst = ((value - exact).abs() / allowed).max().item()
        ulps = ((value - exact).abs() / (magnitude * 2.0 ** -24)).max().item()
        print(f"    {name}: {worst:.3g} x (stated tolerance + 4 ulp of the summed magnitudes); error at most {ulps:.3g} ulp of them")
        assert worst <= 1.0, f"{what}: {name} is {worst:.3g} x the allowance"


def test_synaptic_lif_decay_gradients_against_float64(mods):
    """The C5 configuration (tau_syn 5, tau_mem 20, clamp at -1, at most 2 spikes, 2000 steps) on 512 neurons."""
    hip, ref = mods
    B, T, M = 2, 2000, 256
    n = B * M
    am, asyn = math.exp(-1 / 20.0), math.exp(-1 / 5.0)
    x = (torch.randn(B, T, M, generator=gen(71)) * 0.5 + 0.05)
    go = torch.randn(B, T, M, generator=gen(72))
    dev = "cuda"
    full = lambda v: torch.full((n,), v, device=dev)
    a_mem, a_syn, lo, one, zero = full(am), full(asyn), full(-1.0), full(1.0), full(0.0)
    f = hip.layerLifForward(x.to(dev), zero, zero, a_mem, a_syn, one, one, lo, True, 2, True, True)
    _, gam, gas, _, _ = hip.layerLifBackward(go.to(dev), None, None, x.to(dev), f["ckpt_v"], f["ckpt_i"], zero, zero, a_mem,
                                             a_syn, one, one, lo, True, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    # the fp32 oracle, composed as the reference layer composes it (rows = batch x neurons, time contiguous)
    rows = lambda z: z.movedim(1, 2).reshape(n, T).contiguous()
    xs, gos = rows(x), rows(go)
    r = lambda v: torch.full((n,), v)
    i_rows = ref.leaky_forward((xs * asyn).contiguous(), r(0.0), r(asyn))
    ws, wv = ref.integrate_and_fire_forward(((1.0 - r(am)[:, None]) * i_rows).contiguous(), r(am), r(0.0), r(1.0), None,
                                            r(-1.0), 2)
    assert torch.equal(rows(f["spikes"].cpu()), ws) and ws.sum() > 0
    surr_fn = ref.SingleExponential()
    g_u, g_am_lif, _ = ref.integrate_and_fire_backward(gos, None, wv, ws, r(0.0), r(am), r(1.0), r(1.0), r(-1.0), surr_fn,
                                                       True, gate_initial=True)
    g_i = ((1.0 - r(am)[:, None]) * g_u).contiguous()
    g_xin, g_as_leaky, _ = ref.leaky_integrator_backward(g_i, i_rows, r(0.0), r(asyn), True)
    oracle_gam = g_am_lif - (g_u * i_rows).sum(1)
    oracle_gas = g_as_leaky + (g_xin * xs).sum(1)
    # float64: the same recurrences and sums in double, on the same fp32 forward values
    surr = surr_fn(wv, torch.ones(n, 1)).double()
    nc = (wv > -1.0).double()
    lam64, gam_lif64, _ = ref.lif_backward_recurrence_f64(surr, surr * gos.double(), nc, r(am), r(1.0), v_post=wv - ws,
                                                          v_post_init=r(0.0))
    gam64 = gam_lif64 - (lam64 * i_rows.double()).sum(1)          # norm_input: u = (1 - alpha_mem) i
    mu = torch.zeros(n, dtype=torch.float64)
    gas64 = torch.zeros(n, dtype=torch.float64)
    k = 1.0 - am
    i64, x64 = i_rows.double(), xs.double()
    for t in range(T - 1, -1, -1):
        mu = asyn * mu + k * lam64[:, t]                           # adjoint of i_t
        prev = i64[:, t - 1] if t > 0 else torch.zeros(n, dtype=torch.float64)
        gas64 += mu * (prev + x64[:, t])                           # d i_t / d alpha_syn = i_{t-1} + x_t  (decay_early)
    judge("grad alpha_mem, synaptic LIF, 2000 steps", gam, oracle_gam, gam64)
    judge("grad alpha_syn, synaptic LIF, 2000 steps", gas, oracle_gas, gas64)


def test_leaky_decay_gradient_against_float64(mods):
    """The C3 configuration (ExpLeak, per-channel tau ~ U[5, 50], 1000 steps, gradient of ones) on 1024 rows, through the
    layer kernel and through the (rows, time) kernel."""
    hip, ref = mods
    B, T, M = 4, 1000, 256
    n = B * M
    x = torch.randn(B, T, M, generator=gen(73))
    alpha_c = torch.exp(-1.0 / (5.0 + 45.0 * torch.rand(M, generator=gen(74))))
    alpha = alpha_c.repeat(B)
    dev = "cuda"
    zero = torch.zeros(n, device=dev)
    out, _ = hip.layerLeakyForward(x.to(dev), zero, alpha.to(dev), False, False)
    go = torch.ones(B, T, M)
    _, ga_layer, _ = hip.layerLeakyBackward(go.to(dev), None, out, None, zero, alpha.to(dev), False, False, True)
    rows = lambda z: z.movedim(1, 2).reshape(n, T).contiguous()
    xs, gos = rows(x), rows(go)
    out_rows = ref.leaky_forward(xs, torch.zeros(n), alpha)
    assert torch.equal(rows(out.cpu()), out_rows)
    _, ga_rows, _ = hip.leakyBackwardFused(gos.to(dev), alpha.to(dev), output=out_rows.to(dev), vmemInitial=zero,
                                           needAlphaGrad=True)
    oracle = ref.leaky_backward_alpha(gos, out_rows, torch.zeros(n), alpha)
    g = torch.zeros(n, dtype=torch.float64)
    exact = torch.zeros(n, dtype=torch.float64)
    magnitude = torch.zeros(n, dtype=torch.float64)
    a64, o64 = alpha.double(), out_rows.double()
    for t in range(T - 1, -1, -1):
        g = a64 * g + gos[:, t].double()
        if t > 0:
            exact += g * o64[:, t - 1]
            magnitude += (g * o64[:, t - 1]).abs()
    judge("grad alpha, leaky layer kernel, 1000 steps", ga_layer, oracle, exact, magnitude)
    judge("grad alpha, leaky (rows, time) kernel, 1000 steps", ga_rows, oracle, exact, magnitude)
