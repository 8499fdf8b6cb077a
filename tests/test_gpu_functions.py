"""The autograd Functions on the GPU against the sinabs-style CPU step loop.

Mirrors reference tests/test_spike_functions.py and tests/test_leak_functions.py with the
oracle's per-time-step torch loop (autograd BPTT) in the role that upstream sinabs plays there:
three chained calls carrying state, per-neuron parameters, gradients with respect to input,
initial state and alpha.  Tolerances: fp32 v_mem and gradients rtol 1e-4 / atol 1e-5; spikes
bit-exact except at exact-threshold ties, whose fraction is printed.
"""
from itertools import product

import pytest
import torch

from _util import assert_close, gen, spike_tie_report

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fns():
    assert torch.cuda.is_available()
    from sinabs.exodus.leaky import LeakyIntegrator
    from sinabs.exodus.spike import IntegrateAndFire
    return IntegrateAndFire, LeakyIntegrator


@pytest.fixture(scope="module")
def oracle():
    from oracle import exodus_ref, sinabs_cpu
    return exodus_ref, sinabs_cpu


_g = gen(123)
v_mem_initials = (torch.zeros(2), torch.rand(2, generator=_g) - 0.5)
alphas = (torch.ones(2) * 0.9, torch.rand(2, generator=_g))
thresholds = (torch.ones(2), torch.tensor([0.3, 0.9]))
min_v_mems = (None, -torch.ones(2), torch.tensor([-0.3, -0.4]), torch.tensor([1.2, 0]))
membrane_subtracts = (None, torch.tensor([0.1, 0.2]))
argnames = "v_mem_initial,alpha,threshold,min_v_mem,membrane_subtract"


class CustomSurrogate:
    """A callable the kernels do not know: forces the evaluate-with-torch path."""

    def __call__(self, v_mem, threshold):
        return 1.0 / (1.0 + (v_mem - threshold) ** 2)


@pytest.mark.parametrize(argnames, list(product(v_mem_initials, alphas, thresholds, min_v_mems, membrane_subtracts)))
def test_integratefire(fns, oracle, v_mem_initial, alpha, threshold, min_v_mem, membrane_subtract):
    IntegrateAndFire, _ = fns
    ref, _ = oracle
    inp = torch.rand((2, 10), generator=gen(1)).cuda().requires_grad_(True)
    surrogate = ref.Heaviside(0)
    d = lambda x: None if x is None else x.cuda()
    if membrane_subtract is None:
        membrane_subtract = threshold

    def apply():
        return IntegrateAndFire.apply(inp, d(alpha), d(v_mem_initial), d(threshold), d(membrane_subtract),
                                      d(min_v_mem), surrogate)

    if min_v_mem is not None and (min_v_mem >= threshold).any():
        with pytest.raises(ValueError):
            apply()
    else:
        out, v_mem = apply()
        out.sum().backward()
        assert inp.grad is not None and torch.isfinite(inp.grad).all()
        out, v_mem = apply()
        v_mem.sum().backward()
        assert torch.isfinite(inp.grad).all()
        ws, wv = ref.integrate_and_fire_forward(inp.detach().cpu(), alpha, v_mem_initial, threshold,
                                                membrane_subtract, min_v_mem, None)
        assert torch.equal(out.cpu(), ws) and torch.equal(v_mem.detach().cpu(), wv)


def test_integratefire_argument_errors(fns, oracle):
    IntegrateAndFire, _ = fns
    ref, _ = oracle
    ok = dict(inp=torch.rand(2, 10).cuda(), alpha=torch.full((2,), 0.9).cuda(), v0=torch.zeros(2).cuda(),
              th=torch.ones(2).cuda(), c=torch.ones(2).cuda())

    def call(**kw):
        a = {**ok, **kw}
        return IntegrateAndFire.apply(a["inp"], a["alpha"], a["v0"], a["th"], a["c"], None, ref.Heaviside())

    call()
    with pytest.raises(ValueError, match="2D"):
        call(inp=torch.rand(2, 10, 1).cuda())
    with pytest.raises(ValueError, match="contiguous"):
        call(inp=torch.rand(10, 2).cuda().t())
    with pytest.raises(ValueError, match="1D"):
        call(alpha=torch.full((2, 1), 0.9).cuda())
    with pytest.raises(ValueError, match="between 0 and 1"):
        call(alpha=torch.tensor([0.5, 1.5]).cuda())
    with pytest.raises(ValueError, match="between 0 and 1"):
        call(alpha=torch.tensor([-0.1, 0.5]).cuda())
    with pytest.raises(ValueError, match="1D"):
        call(th=torch.ones(2, 1).cuda())
    with pytest.raises(RuntimeError):                    # CPU tensors: no CPU path
        IntegrateAndFire.apply(torch.rand(2, 10), torch.full((2,), 0.9), torch.zeros(2), torch.ones(2),
                               torch.ones(2), None, ref.Heaviside())


def evolve_exodus(IntegrateAndFire, data, alpha, v_mem_init, threshold, min_v_mem, surrogate_grad_fn,
                  max_num_spikes_per_bin, membrane_subtract):
    """What the layer does around the Function (reference tests/test_spike_functions.py:149-195)."""
    batchsize, timesteps, *trailing = data.shape[1:]
    shape = (batchsize, *trailing)
    ex = lambda p: p.expand(shape).flatten().contiguous()
    alpha = ex(alpha); v_mem_init = ex(v_mem_init); threshold = ex(threshold)
    min_v_mem = None if min_v_mem is None else ex(min_v_mem)
    membrane_subtract = threshold if membrane_subtract is None else ex(membrane_subtract)
    for inp in data:
        inp = inp.movedim(1, -1).reshape(-1, timesteps)
        spikes, v_mem = IntegrateAndFire.apply(inp.contiguous(), alpha, v_mem_init, threshold, membrane_subtract,
                                               min_v_mem, surrogate_grad_fn, max_num_spikes_per_bin)
        v_mem = v_mem - membrane_subtract.unsqueeze(1) * spikes
        v_mem_init = v_mem[:, -1].contiguous()
    return (spikes.reshape(batchsize, *trailing, timesteps).movedim(-1, 1), v_mem[:, -1].reshape(batchsize, *trailing),
            v_mem)


def evolve_steploop(sc, data, alpha, v_mem_init, threshold, min_v_mem, surrogate_grad_fn, max_num_spikes_per_bin,
                    membrane_subtract, clip_mode):
    state = {"v_mem": v_mem_init}
    for inp in data:
        out, state, rec = sc.lif_forward(inp, alpha, None, state, threshold, membrane_subtract, surrogate_grad_fn,
                                         max_num_spikes_per_bin, min_v_mem, norm_input=False, clip_mode=clip_mode)
    return out, state["v_mem"], rec


SURR = ["periodic", "single", "heaviside", "custom"]


def _integratefire_cases():
    """The reference's grid (tests/test_spike_functions.py) in full for the surrogate its test uses; for the
    other surrogates every configuration with a loss on spikes and potential together, and every fifth
    configuration with a loss on the spikes alone and on the potential alone."""
    grid = list(product(v_mem_initials, alphas, thresholds, min_v_mems[:-1], membrane_subtracts))
    cases = [("periodic", *cfg, var) for cfg in grid for var in ("spikes", "vmem", "sum")]
    for name in SURR[1:]:
        cases += [(name, *cfg, "sum") for cfg in grid]
        cases += [(name, *cfg, var) for cfg in grid[SURR.index(name)::5] for var in ("spikes", "vmem")]
    return cases


@pytest.mark.parametrize("surr_name," + argnames + ",backward_var", _integratefire_cases())
def test_compare_integratefire(fns, oracle, surr_name, v_mem_initial, alpha, threshold, min_v_mem, membrane_subtract,
                               backward_var):
    IntegrateAndFire, _ = fns
    ref, sc = oracle
    fn = {"periodic": ref.PeriodicExponential(), "single": ref.SingleExponential(), "heaviside": ref.Heaviside(0.6),
          "custom": CustomSurrogate()}[surr_name]
    if surr_name != "custom":
        # hand the Function an object it recognises as one of the sinabs.activation classes
        from sinabs.exodus._compat import activation as ca
        fn_dev = {"periodic": ca.PeriodicExponential(), "single": ca.SingleExponential(),
                  "heaviside": ca.Heaviside(0.6)}[surr_name]
    else:
        fn_dev = fn
    time_steps, batchsize, n_neurons, num_epochs, cap = 100, 10, 2, 3, 2
    g = gen(1)
    data = torch.rand((num_epochs, batchsize, time_steps, n_neurons), generator=g)

    in_o = data.clone().requires_grad_(True)
    v0_o = v_mem_initial.clone().requires_grad_(True)
    a_o = alpha.clone().requires_grad_(True)
    in_x = data.clone().cuda().requires_grad_(True)
    v0_x = v_mem_initial.clone().cuda().requires_grad_(True)
    a_x = alpha.clone().cuda().requires_grad_(True)
    d = lambda x: None if x is None else x.cuda()

    out_x, vlast_x, _ = evolve_exodus(IntegrateAndFire, in_x, a_x, v0_x, d(threshold), d(min_v_mem), fn_dev, cap,
                                      d(membrane_subtract))
    # clamp written as max(v, lo): the arithmetic of the device code, so spikes must agree exactly
    out_o, vlast_o, _ = evolve_steploop(sc, in_o, a_o, v0_o.expand(batchsize, n_neurons), threshold, min_v_mem, fn,
                                        cap, membrane_subtract, "max")
    assert torch.equal(out_x.detach().cpu(), out_o.detach())
    assert_close(vlast_x, vlast_o, "final v_mem", rtol=1e-4, atol=1e-8 + 1e-6)

    wg = gen(2)
    if backward_var == "spikes":
        w = torch.rand(out_o.shape, generator=wg)
        (w.cuda() * out_x).sum().backward(); (w * out_o).sum().backward()
    elif backward_var == "vmem":
        w = torch.rand(vlast_o.shape, generator=wg)
        (w.cuda() * vlast_x).sum().backward(); (w * vlast_o).sum().backward()
    else:
        w1 = torch.rand(out_o.shape, generator=wg); w2 = torch.rand(vlast_o.shape, generator=wg)
        (out_x * w1.cuda() + (vlast_x * w2.cuda()).unsqueeze(1)).sum().backward()
        (out_o * w1 + (vlast_o * w2).unsqueeze(1)).sum().backward()

    assert_close(in_x.grad, in_o.grad, "grad input")
    assert_close(v0_x.grad, v0_o.grad, "grad v_mem_init", atol=1e-5 * batchsize ** 0.5)
    assert_close(a_x.grad, a_o.grad, "grad alpha", atol=1e-5 * (batchsize * time_steps) ** 0.5)


def test_spikes_against_relu_clamp_are_exact_up_to_ties(fns, oracle, capsys):
    """Upstream-style clamp relu(v-lo)+lo rounds differently on unclipped steps; report the tie fraction."""
    IntegrateAndFire, _ = fns
    ref, sc = oracle
    g = gen(77)
    b, t, m = 64, 300, 64
    data = (torch.randn(1, b, t, m, generator=g) * 0.3 + 0.1)
    alpha = torch.exp(-1 / torch.tensor(20.0)).expand(m).contiguous(); th = torch.ones(m); lo = -torch.ones(m)
    out_x, _, vm_x = evolve_exodus(IntegrateAndFire, data.cuda(), alpha.cuda(), torch.zeros(m).cuda(), th.cuda(),
                                   lo.cuda(), ref.SingleExponential(), 1, None)
    out_o, _, rec = evolve_steploop(sc, data, alpha, torch.zeros(b, m), th, lo, ref.SingleExponential(), 1, None, "relu")
    rows = lambda x: x.movedim(1, -1).reshape(-1, t)
    tie_frac, bad = spike_tie_report(rows(out_x), rows(out_o), rows(rec["v_mem"]), th.expand(b, m).flatten())
    with capsys.disabled():
        print(f"\n[tie report] rows differing through an exact-threshold tie: {tie_frac:.3%}; otherwise: {bad}")
    assert bad == 0


def test_leakyintegrator_smoke(fns):
    _, LeakyIntegrator = fns
    g = gen(1)
    inp = torch.rand((2, 10), generator=g).cuda().requires_grad_(True)
    v0 = torch.zeros(2, device="cuda", requires_grad=True)
    alpha = torch.rand(2, generator=g).cuda().requires_grad_(True)
    LeakyIntegrator.apply(inp, alpha, v0).sum().backward()
    for p in (inp, alpha, v0):
        assert p.grad is not None
    with pytest.raises(ValueError, match="2D"):
        LeakyIntegrator.apply(inp.detach()[0], alpha, v0)
    with pytest.raises(ValueError, match="contiguous"):
        LeakyIntegrator.apply(torch.rand(10, 2).cuda().t(), alpha, v0)


def test_compare_leakyintegrator_backward(fns, oracle):
    _, LeakyIntegrator = fns
    ref, sc = oracle
    time_steps, batchsize, n_neurons, num_epochs = 100, 10, 8, 3
    g = gen(1)
    data = torch.rand((num_epochs, batchsize, time_steps, n_neurons), generator=g)
    v0 = torch.rand(batchsize, n_neurons, generator=g); alpha = torch.rand(n_neurons, generator=g)

    in_o = data.clone().requires_grad_(True); v0_o = v0.clone().requires_grad_(True); a_o = alpha.clone().requires_grad_(True)
    in_x = data.clone().cuda().requires_grad_(True); v0_x = v0.clone().cuda().requires_grad_(True)
    a_x = alpha.clone().cuda().requires_grad_(True)

    # exodus side (reference tests/test_leak_functions.py:78-96)
    a_rows = a_x.expand(v0_x.shape).flatten().contiguous(); state = v0_x.flatten().contiguous()
    for inp in in_x:
        out_x = LeakyIntegrator.apply(inp.movedim(1, -1).reshape(-1, time_steps).contiguous(), a_rows, state)
        state = out_x[:, -1].contiguous()
    out_x = out_x.reshape(batchsize, n_neurons, time_steps).movedim(-1, 1)
    # step loop side
    st = {"v_mem": v0_o}
    for inp in in_o:
        out_o, st, _ = sc.lif_forward(inp, a_o, None, st, None, None, None, None, None, False, spiking=False)

    assert torch.equal(out_x.detach().cpu(), out_o.detach())
    w = torch.rand(out_o.shape, generator=gen(3))
    (w.cuda() * out_x).sum().backward(); (w * out_o).sum().backward()
    assert_close(in_x.grad, in_o.grad, "grad input", rtol=1e-5, atol=1e-6)
    assert_close(v0_x.grad, v0_o.grad, "grad v_init", rtol=1e-5, atol=1e-6)
    assert_close(a_x.grad, a_o.grad, "grad alpha", rtol=1e-4, atol=1e-4)


def test_deferred_parameter_validation(fns, oracle):
    """In 'deferred' mode a bad alpha does not stop the call that carries it; the error surfaces at
    flush() (or at a later call), and good parameters never raise."""
    IntegrateAndFire, _ = fns
    ref, _ = oracle
    from sinabs.exodus import _validate as val
    x = torch.rand(2, 10).cuda(); one = torch.ones(2).cuda(); zero = torch.zeros(2).cuda()
    try:
        val.set_mode("deferred")
        IntegrateAndFire.apply(x, one * 0.9, zero, one, one, None, ref.Heaviside())
        val.flush()
        IntegrateAndFire.apply(x, torch.tensor([0.5, 1.5]).cuda(), zero, one, one, None, ref.Heaviside())
        with pytest.raises(ValueError, match="between 0 and 1"):
            val.flush()
        IntegrateAndFire.apply(x, one * 0.9, zero, one, one, -one * 2, ref.Heaviside())
        IntegrateAndFire.apply(x, one * 0.9, zero, one, one, one * 2, ref.Heaviside())
        with pytest.raises(ValueError, match="greater than"):
            val.flush()
    finally:
        val.set_mode("sync")
