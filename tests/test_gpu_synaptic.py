"""The fused synapse + membrane Function against (a) the composition of the two separate
Functions, as the reference layer chains them, and (b) autograd through the CPU step loop."""
import pytest
import torch

from _util import assert_close, gen, spike_tie_report

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    assert torch.cuda.is_available()
    from sinabs.exodus._compat import activation as act
    from sinabs.exodus.leaky import LeakyIntegrator
    from sinabs.exodus.spike import IntegrateAndFire
    from sinabs.exodus.synaptic import SynapticIntegrateAndFire
    return act, LeakyIntegrator, IntegrateAndFire, SynapticIntegrateAndFire


def composed(LeakyIntegrator, IntegrateAndFire, x, a_syn, a_mem, i0, v0, th, c, lo, fn, cap, decay_early, norm_input):
    """reference sinabs/exodus/layers/lif.py:185-254"""
    xin = x * a_syn.unsqueeze(1) if decay_early else x
    i_syn = LeakyIntegrator.apply(xin.contiguous(), a_syn, i0)
    u = (1.0 - a_mem.unsqueeze(1)) * i_syn if norm_input else i_syn
    s, v = IntegrateAndFire.apply(u.contiguous(), a_mem, v0, th, c, lo, fn, cap)
    return s, v, i_syn


@pytest.mark.parametrize("n,t", [(3, 7), (70, 100), (300, 301), (1000, 64)])
@pytest.mark.parametrize("surr", ["single", "periodic", "heaviside"])
@pytest.mark.parametrize("decay_early,norm_input,use_lo,cap,extra",
                         [(True, True, True, 2, False), (False, True, False, None, True),
                          (True, False, True, 1, True), (False, False, False, 3, False)])
def test_fused_equals_composed(mods, n, t, surr, decay_early, norm_input, use_lo, cap, extra):
    act, Leaky, IAF, Fused = mods
    fn = {"single": act.SingleExponential(), "periodic": act.PeriodicExponential(0.4, 0.8),
          "heaviside": act.Heaviside(0.7)}[surr]
    g = gen(n * 31 + t)
    mk = lambda *shape, s=1.0, o=0.0: (torch.randn(*shape, generator=g) * s + o).cuda()
    x = mk(n, t, s=0.8, o=0.3)
    a_syn = (0.1 + 0.8 * torch.rand(n, generator=g)).cuda(); a_mem = (0.1 + 0.9 * torch.rand(n, generator=g)).cuda()
    i0 = mk(n, s=0.3); v0 = mk(n, s=0.3)
    th = (0.5 + torch.rand(n, generator=g)).cuda(); c = (0.3 + 0.5 * torch.rand(n, generator=g)).cuda()
    lo = (-0.3 - 0.3 * torch.rand(n, generator=g)).cuda() if use_lo else None
    w = [mk(n, t) for _ in range(3)]

    leaves_a = [p.clone().requires_grad_(True) for p in (x, a_syn, a_mem, i0, v0)]
    leaves_b = [p.clone().requires_grad_(True) for p in (x, a_syn, a_mem, i0, v0)]
    sa, va, ia = Fused.apply(leaves_a[0], leaves_a[1], leaves_a[2], leaves_a[3], leaves_a[4], th, c, lo, fn, cap,
                             decay_early, norm_input)
    sb, vb, ib = composed(Leaky, IAF, leaves_b[0], leaves_b[1], leaves_b[2], leaves_b[3], leaves_b[4], th, c, lo, fn,
                          cap, decay_early, norm_input)
    assert torch.equal(ia, ib) and torch.equal(va, vb) and torch.equal(sa, sb)

    def loss(s, v, i):
        l = (s * w[0]).sum()
        if extra:
            l = l + (v * w[1]).sum() + (i * w[2]).sum()
        return l

    loss(sa, va, ia).backward(); loss(sb, vb, ib).backward()
    names = ("input", "alpha_syn", "alpha_mem", "i_syn_init", "v_mem_init")
    for nm, pa, pb in zip(names, leaves_a, leaves_b):
        atol = 1e-5 * (t ** 0.5 if nm.startswith("alpha") else 1.0)
        assert_close(pa.grad, pb.grad, f"grad {nm}", rtol=1e-4, atol=atol)


def test_fused_against_cpu_step_loop(mods, capsys):
    """sinabs-style loop: i = a_syn*(i + x); v = a_mem*v_post + (1-a_mem)*i; autograd BPTT."""
    act, _, _, Fused = mods
    from oracle import exodus_ref as ref
    from oracle import sinabs_cpu as sc
    b, t, m = 4, 200, 96
    g = gen(5)
    x = torch.randn(b, t, m, generator=g) * 0.5 + 0.05
    a_s = torch.full((m,), 0.8187); a_m = torch.full((m,), 0.9512)
    xo = x.clone().requires_grad_(True); aso = a_s.clone().requires_grad_(True); amo = a_m.clone().requires_grad_(True)
    out, state, rec = sc.lif_forward(xo, amo, aso, {"v_mem": torch.zeros(b, m), "i_syn": torch.zeros(b, m)}, 1.0, None,
                                     ref.SingleExponential(), 2, -1.0, True, clip_mode="max")
    out.sum().backward()

    rows = lambda p: p.expand(b, m).flatten().contiguous().cuda()
    xd = sc.bt_to_rows(x).cuda().requires_grad_(True)
    asd = a_s.clone().cuda().requires_grad_(True); amd = a_m.clone().cuda().requires_grad_(True)
    ex = lambda p: p.expand(b, m).flatten().contiguous()
    z = torch.zeros(b * m, device="cuda")
    s, v, i = Fused.apply(xd, ex(asd), ex(amd), z, z, rows(torch.ones(m)), None, rows(-torch.ones(m)),
                          act.SingleExponential(), 2, True, True)
    s.sum().backward()

    # a_syn*(i+x) and a_syn*i + a_syn*x round differently: potentials agree to fp32 tolerance and
    # spike trains up to rows that hit a threshold tie
    tie, bad = spike_tie_report(s, sc.bt_to_rows(out), sc.bt_to_rows(rec["v_mem"]), torch.ones(b * m), ulps=64)
    with capsys.disabled():
        print(f"\n[tie report, synaptic LIF] rows differing through a threshold tie: {tie:.3%}; otherwise: {bad}")
    assert bad == 0
    if tie == 0:
        assert_close(v, sc.bt_to_rows(rec["v_mem"]), "v_mem", rtol=1e-4, atol=1e-5)
        assert_close(xd.grad, sc.bt_to_rows(xo.grad), "grad input", rtol=1e-4, atol=1e-5)
        assert_close(asd.grad, aso.grad, "grad alpha_syn", rtol=1e-4, atol=1e-5)
        assert_close(amd.grad, amo.grad, "grad alpha_mem", rtol=1e-4, atol=1e-5)
