"""The layer-layout kernels (whole layer on (batch, time, neurons), recompute-in-backward) against
the (rows, time) path of the same layer and against the CPU oracle."""
from itertools import product

import pytest
import torch

from _util import assert_close, gen

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["one lane per neuron", "small layers split over time"])
def backward_kernel_choice(request):
    """Every test of this file runs twice: with the backward kernel that walks a neuron's sequence in one lane only, and
    with the default choice, which hands small layers to the kernel that gives every 32 steps a lane."""
    from sinabs.exodus import _hip
    before = _hip.backwardTimeSplit(0 if request.param.startswith("one") else 1)
    yield
    _hip.backwardTimeSplit(before)


@pytest.fixture(scope="module")
def L():
    assert torch.cuda.is_available()
    import sinabs.exodus.layers as el
    from sinabs.exodus import _hip
    from sinabs.exodus._compat import activation as act
    return el, act, _hip


def pair(el, cls, **kw):
    a = cls(**kw).cuda(); b = cls(**kw).cuda()
    b.native_layout = False
    return a, b


SHAPES = [(1, 1, (1,)), (2, 7, (3,)), (3, 33, (5, 4)), (2, 100, (2, 7, 7)), (4, 64, (256,)), (2, 300, (260,)),
          (3, 97, (1024,))]


@pytest.mark.parametrize("batch,steps,trailing", SHAPES)
@pytest.mark.parametrize("tau_syn,decay_early,norm_input", [(None, True, True), (None, True, False), (6.0, True, True),
                                                             (6.0, False, False)])
@pytest.mark.parametrize("spike,lo,surr", [("multi", None, "single"), ("max2", -0.7, "periodic"), ("single", -0.3, "heaviside")])
def test_native_equals_rows_path(L, batch, steps, trailing, tau_syn, decay_early, norm_input, spike, lo, surr):
    el, act, _ = L
    m = 1
    for d in trailing:
        m *= d
    fn = {"multi": act.MultiSpike, "single": act.SingleSpike, "max2": act.MaxSpike(2)}[spike]
    sg = {"single": act.SingleExponential(), "periodic": act.PeriodicExponential(0.4, 0.8), "heaviside": act.Heaviside(0.7)}[surr]
    g = gen(batch * 1000 + steps + m)
    kw = dict(tau_mem=10.0 + 20.0 * torch.rand(trailing, generator=g), tau_syn=tau_syn, spike_fn=fn, min_v_mem=lo,
              surrogate_grad_fn=sg, train_alphas=True, norm_input=norm_input, decay_early=decay_early)
    native, rows = pair(el, el.LIF, **kw)
    scale = (8.0 if norm_input else 0.8) * (1.0 if tau_syn is None else 0.4)
    data = (torch.rand((2, batch, steps) + trailing, generator=g) * scale * 2 - 0.3 * scale).cuda()
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    for k in range(2):                                   # second call starts from the first call's states
        a = native(xa[k]); b = rows(xb[k])
        assert a.shape == b.shape == xa[k].shape
        assert torch.equal(a, b)
        assert torch.equal(native.v_mem, rows.v_mem)
        if tau_syn is not None:
            assert torch.equal(native.i_syn, rows.i_syn)
        assert torch.allclose(native.firing_rate, rows.firing_rate, rtol=1e-6, atol=0)
    w = torch.rand(a.shape, generator=g).cuda()
    (a * w).sum().backward(); (b * w).sum().backward()
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(native.named_parameters(), rows.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-5 * max(1.0, (batch * steps) ** 0.5))


def test_native_iaf_squeeze_callable_surrogate_and_records(L):
    el, act, _ = L
    x = torch.rand(6 * 50, 2, 5, 5, generator=gen(3)).cuda()
    native, rows = pair(el, el.IAFSqueeze, batch_size=6, min_v_mem=-1.0)
    assert torch.equal(native(x), rows(x)) and native(x).is_contiguous()
    custom = el.IAF(surrogate_grad_fn=lambda v, th: 1.0 / (1.0 + (v - th) ** 2)).cuda()
    xg = x.reshape(6, 50, 2, 5, 5).clone().requires_grad_(True)
    assert custom._use_native_layout(xg)                              # any callable runs on the layer kernels
    rec = el.IAF(record_states=True).cuda()
    assert rec._use_native_layout(xg)                                 # and so do differentiable state records
    out = rec(xg); assert out.shape == (6, 50, 2, 5, 5)
    (out.sum() + rec.recordings["v_mem"].sum()).backward()
    assert xg.grad is not None and bool(torch.isfinite(xg.grad).all())


def test_native_forward_against_cpu_oracle(L):
    """Bit-exact spikes and final states against the C restatement of the reference kernel."""
    el, act, hip = L
    from oracle import exodus_ref as ref
    from oracle import sinabs_cpu as sc
    b, t, m = 3, 130, 40
    g = gen(11)
    x = torch.randn(b, t, m, generator=g) * 0.6 + 0.2
    alpha = torch.rand(b * m, generator=g); v0 = torch.randn(b * m, generator=g) * 0.3
    th = 0.5 + torch.rand(b * m, generator=g); c = 0.3 + 0.5 * torch.rand(b * m, generator=g); lo = -0.5 * torch.ones(b * m)
    ws, wv = ref.lif_forward(sc.bt_to_rows(x), v0, alpha, c, th, lo, True, 2)
    D = lambda z: z.cuda()
    res = hip.layerLifForward(D(x), D(v0), None, D(alpha), None, D(c), D(th), D(lo), True, 2, True, False,
                              wantRecords=True)
    assert torch.equal(res["spikes"].cpu(), sc.rows_to_bt(ws, b))
    vpost = wv - c[:, None] * ws
    assert torch.equal(res["v_rec"].cpu(), sc.rows_to_bt(vpost, b))
    assert torch.equal(res["v_last"].cpu(), vpost[:, -1])
    assert float(res["spike_sum"]) == float(ws.sum())
    ck = hip.checkpointInterval()
    want_ck = torch.stack([v0] + [vpost[:, k * ck - 1] for k in range(1, (t + ck - 1) // ck)], 1)   # (rows, n_ck)
    assert torch.equal(res["ckpt_v"].cpu(), sc.rows_to_bt(want_ck, b))


@pytest.mark.parametrize("batch,steps,trailing", [(1, 1, (1,)), (2, 7, (3,)), (3, 33, (5, 4)), (4, 64, (256,)), (2, 300, (260,))])
@pytest.mark.parametrize("decay_early,norm_input,train_alphas", list(product((True, False), (True, False), (True, False))))
def test_native_expleak_equals_rows_path(L, batch, steps, trailing, decay_early, norm_input, train_alphas):
    el, _, _ = L
    g = gen(batch * 100 + steps)
    kw = dict(tau_mem=5.0 + 40.0 * torch.rand(trailing, generator=g), train_alphas=train_alphas, norm_input=norm_input,
              decay_early=decay_early)
    native, rows = pair(el, el.ExpLeak, **kw)
    data = torch.randn((2, batch, steps) + trailing, generator=g).cuda()
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    for k in range(2):
        a = native(xa[k]); b = rows(xb[k])
        assert torch.equal(a, b) and torch.equal(native.v_mem, rows.v_mem)
    w = torch.randn(a.shape, generator=g).cuda()
    (a * w).sum().backward(); (b * w).sum().backward()
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(native.named_parameters(), rows.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-5 * max(1.0, (batch * steps) ** 0.5))


def test_native_expleak_records_and_squeeze(L):
    el, _, _ = L
    x = torch.rand(5 * 40, 3, 4, 4, generator=gen(5)).cuda()
    native, rows = pair(el, el.ExpLeakSqueeze, tau_mem=12.0, batch_size=5, record_states=True)
    a = native(x); b = rows(x)
    assert torch.equal(a, b) and torch.equal(native.recordings["v_mem"], rows.recordings["v_mem"])


@pytest.mark.parametrize("cap", [0, 1, 2, 3, 5, -1])
@pytest.mark.parametrize("b,t,m", [(2, 31, 6), (3, 32, 10), (2, 33, 7), (1, 64, 260), (2, 97, 64), (1, 5, 1), (20, 40, 2048)])
@pytest.mark.parametrize("theta_sign", ["positive", "mixed"])
def test_native_membrane_against_cpu_oracle_all_caps(L, cap, b, t, m, theta_sign):
    """Every spike-count specialisation (cap 1, cap 2, general), every lane width, sequences that
    end inside / at / just after a checkpoint block, and thresholds that are not positive (which take
    the quotient path): spikes and states bit for bit, gradients within tolerance, against the C
    restatement of the reference kernels."""
    _, _, hip = L
    from oracle import exodus_ref as ref
    from oracle import sinabs_cpu as sc
    n = b * m
    g = gen(cap * 1000 + t * 10 + m)
    x = torch.randn(b, t, m, generator=g) * 1.5 + 0.4          # up to ~6 spikes per step
    alpha = 0.3 + 0.7 * torch.rand(n, generator=g); v0 = torch.randn(n, generator=g) * 0.3
    th = 0.5 + torch.rand(n, generator=g); c = 0.3 + 0.5 * torch.rand(n, generator=g)
    lo = -0.5 - torch.rand(n, generator=g)
    if theta_sign == "mixed":
        th[::3] = -th[::3] * 0.2                               # still above the lower bound
        th[1::7] = 0.0
    ws, wv = ref.lif_forward(sc.bt_to_rows(x), v0, alpha, c, th, lo, True, cap)
    D = lambda z: z.cuda()
    res = hip.layerLifForward(D(x), D(v0), None, D(alpha), None, D(c), D(th), D(lo), True, cap, True, False)
    assert torch.equal(res["spikes"].cpu(), sc.rows_to_bt(ws, b))
    vpost = wv - c[:, None] * ws
    assert torch.equal(res["v_last"].cpu(), vpost[:, -1])
    total = float(ws.double().sum())                       # a zero threshold without cap gives 2^32 - 1 "spikes"
    assert abs(float(res["spike_sum"]) - total) <= 1e-6 * total
    if cap > 0:
        assert ws.max() <= cap
    if theta_sign == "mixed":
        return                                                 # surrogates divide by the threshold
    go = torch.randn(b, t, m, generator=g)
    gi, ga, gv0 = ref.integrate_and_fire_backward(sc.bt_to_rows(go), None, wv, ws, v0, alpha, c, th, lo,
                                                  ref.SingleExponential(), True, gate_initial=True)
    got = hip.layerLifBackward(D(go), None, None, D(x), res["ckpt_v"], None, D(v0), None, D(alpha), None, D(c),
                               D(th), D(lo), True, cap, True, False, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    from _util import assert_close_rowscaled
    assert_close_rowscaled(sc.bt_to_rows(got[0].cpu()), gi, "grad input")
    assert_close(got[3].cpu(), gv0, "grad v_init", atol=1e-5 * max(1.0, gv0.abs().max().item()))
    assert_close(got[1].cpu(), ga, "grad alpha", rtol=2e-4, atol=2e-5 * max(1.0, ga.abs().max().item()))


@pytest.mark.parametrize("cap", [1, 2, -1])
@pytest.mark.parametrize("b,t,m", [(2, 31, 6), (3, 32, 10), (2, 33, 7), (2, 97, 67), (1, 64, 260), (3, 97, 1030)])
@pytest.mark.parametrize("decay_early,norm_input", list(product((True, False), (True, False))))
def test_native_synaptic_against_cpu_oracle(L, cap, b, t, m, decay_early, norm_input):
    """The synaptic layer kernels (the benchmark's kernels) directly against the CPU oracle, composed the
    way the reference layer composes its Functions: both input options, the three spike-count
    specialisations, sequences that end inside / at / just after a checkpoint block, ragged widths,
    random per-neuron parameters and initial states, gradients arriving at spikes and at both final
    states.  Forward bit for bit; gradients of input, both decay factors and both initial states within
    rtol 1e-4 / atol 1e-5 (sums over time: atol scaled by sqrt(t), worst error printed in plain units)."""
    _, _, hip = L
    from oracle import exodus_ref as ref
    from oracle import sinabs_cpu as sc
    from _util import synaptic_layer_oracle, worst
    n = b * m
    g = gen(7000 + cap * 100 + t * 10 + m + 2 * decay_early + norm_input)
    scale = (6.0 if norm_input else 0.7) * 0.5
    x = torch.randn(b, t, m, generator=g) * scale + 0.3 * scale
    am = 0.5 + 0.5 * torch.rand(n, generator=g); asn = 0.3 + 0.6 * torch.rand(n, generator=g)
    v0 = torch.randn(n, generator=g) * 0.3; i0 = torch.randn(n, generator=g) * 0.3
    th = 0.5 + torch.rand(n, generator=g); c = th * (0.4 + 0.6 * torch.rand(n, generator=g))
    lo = -0.2 - torch.rand(n, generator=g)
    go = torch.randn(b, t, m, generator=g); gvl = torch.randn(n, generator=g); gil = torch.randn(n, generator=g)
    want = synaptic_layer_oracle(ref, sc.bt_to_rows(x), sc.bt_to_rows(go), am, asn, v0, i0, th, c, lo, cap, decay_early,
                                 norm_input, ref.SingleExponential(), gvl, gil)
    D = lambda z: z.cuda()
    f = hip.layerLifForward(D(x), D(v0), D(i0), D(am), D(asn), D(c), D(th), D(lo), True, cap, decay_early, norm_input)
    assert want["spikes"].sum() > 0
    assert torch.equal(f["spikes"].cpu(), sc.rows_to_bt(want["spikes"], b))
    assert torch.equal(f["v_last"].cpu(), want["v_last"]) and torch.equal(f["i_last"].cpu(), want["i_last"])
    got = hip.layerLifBackward(D(go), D(gvl), D(gil), D(x), f["ckpt_v"], f["ckpt_i"], D(v0), D(i0), D(am), D(asn), D(c),
                               D(th), D(lo), True, cap, decay_early, norm_input, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    gx, g_am, g_as, g_v0, g_i0 = (z.cpu() for z in got)
    assert_close(sc.bt_to_rows(gx), want["g_x"], "grad input")
    assert_close(g_v0, want["g_v_init"], "grad v_init")
    assert_close(g_i0, want["g_i_init"], "grad i_init")
    print(f"alpha_mem grad {worst(g_am, want['g_alpha_mem'])}; alpha_syn grad {worst(g_as, want['g_alpha_syn'])}")
    assert_close(g_am, want["g_alpha_mem"], "grad alpha_mem", atol=1e-5 * t ** 0.5)
    assert_close(g_as, want["g_alpha_syn"], "grad alpha_syn", atol=1e-5 * t ** 0.5)


@pytest.mark.parametrize("kind", ["lif", "synaptic", "expleak"])
def test_firing_rate_carries_gradient_like_the_reference(L, kind):
    """The reference computes ``firing_rate = output.sum() / output.numel()`` with autograd
    (layers/lif.py:305), so a loss on it reaches the input; the kernels hand the sum out as a
    differentiable scalar instead of reading the output again."""
    el, act, _ = L
    kw = dict(tau_mem=12.0, train_alphas=True)
    if kind == "expleak":
        native, rows = pair(el, el.ExpLeak, **kw)
    else:
        native, rows = pair(el, el.LIF, tau_syn=5.0 if kind == "synaptic" else None, min_v_mem=-0.5, **kw)
    data = (torch.rand(3, 45, 70, generator=gen(8)) * 6 - 1).cuda()
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    a = native(xa); b = rows(xb)
    w = torch.rand(a.shape, generator=gen(9)).cuda()
    ((a * w).sum() * 0.01 + 3.0 * native.firing_rate).backward()
    ((b * w).sum() * 0.01 + 3.0 * rows.firing_rate).backward()
    assert torch.allclose(native.firing_rate, rows.firing_rate, rtol=1e-5, atol=1e-7)
    assert xa.grad.abs().sum() > 0
    assert_close(xa.grad, xb.grad, "grad input through firing_rate")
    for (k, p), (_, q) in zip(native.named_parameters(), rows.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=2e-5)


def test_wide_lane_kernels_equal_one_neuron_per_lane(L):
    """Layers large enough for 2 or 4 neurons per lane (8- and 16-byte accesses) against the same
    batch elements computed alone, which is small enough to run with one neuron per lane: bit for bit,
    in every output, on repeated runs (two blocks per compute unit overlap here, which is where a
    store whose data registers are rewritten too early shows up)."""
    _, _, hip = L
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(3)
    full = lambda n, v: torch.full((n,), v, device=dev)

    B, T, M = 4, 40, 131072                                   # leaky: 4 neurons per lane (2 with alpha gradient)
    x = torch.randn(B, T, M, generator=g, device=dev); go = torch.randn(B, T, M, generator=g, device=dev)

    def leaky(xx, gg):
        n = xx.shape[0] * M
        out, v_last = hip.layerLeakyForward(xx, full(n, 0.1), full(n, 0.9), True, True)
        gi, ga, gv = hip.layerLeakyBackward(gg, None, out, xx, full(n, 0.1), full(n, 0.9), True, True, True)
        gi2 = hip.layerLeakyBackward(gg, None, None, None, None, full(n, 0.9), True, True, False)[0]
        return out, gi, gi2, v_last, ga, gv

    for nb in (B, 2):                                          # 4 batch elements: 4 neurons per lane; 2: 2 per lane
        for _ in range(3):
            big = leaky(x[:nb].contiguous(), go[:nb].contiguous())
            for b in range(nb):
                one = leaky(x[b:b + 1].contiguous(), go[b:b + 1].contiguous())
                for p, q in zip(big, one):
                    assert torch.equal(p[b] if p.ndim == 3 else p[b * M:(b + 1) * M], q[0] if q.ndim == 3 else q)

    B, T, M = 8, 40, 65536                                    # spiking forward: 2 neurons per lane
    x = torch.randn(B, T, M, generator=g, device=dev) * 0.8 + 0.2

    def spiking(xx):
        n = xx.shape[0] * M
        f = hip.layerLifForward(xx, full(n, 0.0), full(n, 0.0), full(n, 0.95), full(n, 0.8), full(n, 1.0), full(n, 1.0),
                                full(n, -1.0), True, -1, True, True)
        return f["spikes"], f["v_last"], f["i_last"], f["ckpt_v"]

    for _ in range(3):
        big = spiking(x)
        assert big[0].sum() > 0
        for b in range(B):
            one = spiking(x[b:b + 1].contiguous())
            for p, q in zip(big, one):
                assert torch.equal(p[b] if p.ndim == 3 else p[b * M:(b + 1) * M], q[0] if q.ndim == 3 else q)


def test_random_configurations_forward_against_cpu_oracle(L):
    """A seeded sweep over shapes (every remainder of the 32-step blocks and 16-step stages, odd and
    even neuron counts), options, caps and initial states: spikes, final states and checkpoints bit
    for bit against the oracle composed the way the reference layer composes its Functions."""
    _, _, hip = L
    from oracle import exodus_ref as ref
    from oracle import sinabs_cpu as sc
    import random
    rnd = random.Random(1234)
    D = lambda z: None if z is None else z.cuda()
    for case in range(60):
        b = rnd.choice([1, 2, 3, 5])
        t = rnd.choice([1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 95, 96, 100, 129])
        m = rnd.choice([1, 2, 3, 6, 64, 65, 130, 256, 258, 1000])
        syn = rnd.random() < 0.5
        decay_early = rnd.random() < 0.5
        norm_input = rnd.random() < 0.5
        use_lo = rnd.random() < 0.6
        cap = rnd.choice([-1, 1, 2, 3])
        n = b * m
        g = gen(1000 + case)
        scale = (6.0 if norm_input else 0.7) * (0.5 if syn else 1.0)
        x = torch.randn(b, t, m, generator=g) * scale + 0.3 * scale
        am = 0.5 + 0.5 * torch.rand(n, generator=g); asn = 0.3 + 0.6 * torch.rand(n, generator=g)
        v0 = torch.randn(n, generator=g) * 0.3; i0 = torch.randn(n, generator=g) * 0.3
        th = 0.5 + torch.rand(n, generator=g); c = 0.3 + 0.6 * torch.rand(n, generator=g)
        lo = -0.2 - torch.rand(n, generator=g)
        xr = sc.bt_to_rows(x)
        if syn:
            xin = (xr * asn[:, None]).contiguous() if decay_early else xr
            i_rows = ref.leaky_forward(xin, i0, asn)
        else:
            i_rows = xr
        u = ((1.0 - am)[:, None] * i_rows).contiguous() if norm_input else i_rows
        ws, wv = ref.lif_forward(u, v0, am, c, th, lo if use_lo else None, use_lo, cap)
        res = hip.layerLifForward(D(x), D(v0), D(i0) if syn else None, D(am), D(asn) if syn else None, D(c), D(th),
                                  D(lo) if use_lo else None, use_lo, cap, decay_early, norm_input)
        what = f"case {case}: b={b} t={t} m={m} syn={syn} de={decay_early} norm={norm_input} lo={use_lo} cap={cap}"
        assert torch.equal(res["spikes"].cpu(), sc.rows_to_bt(ws, b)), what
        vpost = wv - c[:, None] * ws
        assert torch.equal(res["v_last"].cpu(), vpost[:, -1]), what
        if syn:
            assert torch.equal(res["i_last"].cpu(), i_rows[:, -1]), what
        ck = hip.checkpointInterval()
        n_ck = (t + ck - 1) // ck
        want_ck = torch.stack([v0] + [vpost[:, k * ck - 1] for k in range(1, n_ck)], 1)
        assert torch.equal(res["ckpt_v"].cpu(), sc.rows_to_bt(want_ck, b)), what
        assert float(res["spike_sum"]) == float(ws.double().sum()), what


def test_empty_sequences_and_batches(L):
    """Zero time steps leave the states where they were; zero batch elements or neurons give empty
    outputs; nothing is launched and nothing faults."""
    el, _, hip = L
    D = lambda z: z.cuda()
    v0 = torch.tensor([0.3, -0.2, 0.7]); i0 = torch.tensor([0.1, 0.2, 0.3]); one = torch.ones(3)
    x = torch.empty(1, 0, 3)
    res = hip.layerLifForward(D(x), D(v0), D(i0), D(one * 0.9), D(one * 0.8), D(one), D(one), None, False, -1, True, True)
    assert res["spikes"].shape == (1, 0, 3) and torch.equal(res["v_last"].cpu(), v0) and torch.equal(res["i_last"].cpu(), i0)
    out, v_last = hip.layerLeakyForward(D(x), D(v0), D(one * 0.9), True, True)
    assert out.shape == (1, 0, 3) and torch.equal(v_last.cpu(), v0)
    for shape in [(0, 5, 3), (2, 5, 0)]:
        n = shape[0] * shape[2]
        e = torch.empty(n)
        res = hip.layerLifForward(D(torch.empty(shape)), D(e), None, D(e), None, D(e), D(e), None, False, -1, True, True)
        assert res["spikes"].shape == shape and res["v_last"].numel() == 0
    layer = el.IAF().cuda()
    assert layer(torch.empty(2, 0, 4).cuda()).shape == (2, 0, 4)
    # backward over zero steps: a gradient on a final state is the gradient of the initial state,
    # the decay factors get zero (nothing is launched, so nothing may be left uninitialised)
    gv = torch.tensor([1.0, -2.0, 3.0]); gi = torch.tensor([0.5, 0.25, -1.0])
    ck = torch.empty(1, 0, 3)
    for _ in range(3):                                         # fresh allocations each time
        torch.full((1 << 16,), float("nan")).cuda()            # dirty memory for the allocator to hand out again
        got = hip.layerLifBackward(D(x), D(gv), D(gi), D(x), D(ck), D(ck), D(v0), D(i0), D(one * 0.9), D(one * 0.8),
                                   D(one), D(one), None, False, -1, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
        assert got[0].shape == (1, 0, 3)
        assert torch.equal(got[1].cpu(), torch.zeros(3)) and torch.equal(got[2].cpu(), torch.zeros(3))
        assert torch.equal(got[3].cpu(), gv) and torch.equal(got[4].cpu(), gi)
    got = hip.layerLifBackward(D(x), None, None, D(x), D(ck), None, D(v0), None, D(one * 0.9), None, D(one), D(one),
                               None, False, -1, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    assert torch.equal(got[3].cpu(), torch.zeros(3)) and got[2] is None and got[4] is None
    # through the layer: a loss on the state after an empty sequence reaches the state before it
    lif = el.LIF(tau_mem=10.0, tau_syn=5.0, train_alphas=True).cuda()
    warm = (torch.rand(2, 5, 4, generator=gen(1)) * 3).cuda().requires_grad_(True)
    lif(warm)                                                  # states now carry a graph
    lif(torch.empty(2, 0, 4).cuda())
    (lif.v_mem.sum() + 2.0 * lif.i_syn.sum()).backward()
    assert warm.grad is not None and bool(torch.isfinite(warm.grad).all()) and bool((warm.grad != 0).any())
    assert bool(torch.isfinite(lif.alpha_mem.grad).all()) and bool(torch.isfinite(lif.alpha_syn.grad).all())


@pytest.mark.parametrize("mode", ["no_grad", "inference_mode", "non_contiguous", "half_input"])
def test_inference_and_unusual_inputs(L, mode):
    """Inference needs no checkpoints and gives the same spikes; a transposed view is made contiguous;
    a half-precision input does not take the float32 kernels' fast path and is refused by the
    (rows, time) Functions the way the reference refuses it (its kernels are float32 only)."""
    el, _, _ = L
    native, rows = pair(el, el.LIF, tau_mem=10.0, tau_syn=5.0, min_v_mem=-1.0)
    x = (torch.rand(3, 40, 50, generator=gen(2)) * 4).cuda()
    want = rows(x)
    if mode == "no_grad":
        with torch.no_grad():
            got = native(x)
        assert not got.requires_grad
    elif mode == "inference_mode":
        with torch.inference_mode():
            got = native(x)
    elif mode == "non_contiguous":
        xt = x.transpose(0, 2).contiguous().transpose(0, 2)   # same values, strides of another layout
        assert not xt.is_contiguous()
        got = native(xt)
    else:
        assert not native._use_native_layout(x.half())
        with pytest.raises((RuntimeError, ValueError, TypeError)):
            native(x.half())
        return
    assert torch.equal(got, want) and torch.equal(native.v_mem, rows.v_mem)


@pytest.mark.parametrize("tau_syn", [None, 5.0])
def test_inference_records_states_and_accepts_any_surrogate(L, tau_syn):
    """Without gradients the layer kernels serve every configuration: they write the per-step states
    themselves (``record_states``) and never evaluate the surrogate."""
    el, act, _ = L
    custom = lambda v, th: 1.0 / (1.0 + (v - th) ** 2)
    kw = dict(tau_mem=12.0, tau_syn=tau_syn, min_v_mem=-0.5, record_states=True, surrogate_grad_fn=custom)
    native, rows = pair(el, el.LIF, **kw)
    x = (torch.rand(3, 70, 5, 8, generator=gen(4)) * 5 - 1).cuda()
    with torch.no_grad():
        assert native._use_native_layout(x)
        for _ in range(2):                                     # second call continues from the first call's states
            a = native(x); b = rows(x)
            assert torch.equal(a, b)
            assert torch.equal(native.recordings["v_mem"], rows.recordings["v_mem"])
            assert torch.equal(native.v_mem, rows.v_mem) and torch.equal(native.recordings["v_mem"][:, -1], native.v_mem)
            if tau_syn is not None:
                assert torch.equal(native.recordings["i_syn"], rows.recordings["i_syn"])
            assert torch.allclose(native.firing_rate, rows.firing_rate, rtol=1e-6, atol=0)
    with pytest.raises(ValueError):
        bad = el.LIF(tau_mem=10.0, min_v_mem=2.0).cuda()
        with torch.no_grad():
            bad(x)


@pytest.mark.parametrize("tau_syn", [None, 6.0])
@pytest.mark.parametrize("shape", [(3, 70, 5, 8), (2, 45, 37)])
def test_any_callable_surrogate_on_the_layer_kernels(L, tau_syn, shape):
    """A surrogate gradient the kernels do not know is evaluated by the caller's function on the recorded
    pre-reset potential and streamed into the backward kernel; gradients equal those of the (rows, time)
    Functions, which call the same function on the same potentials (reference sinabs/exodus/spike.py:251)."""
    el, act, _ = L
    calls = []
    def custom(v, th):
        calls.append((tuple(v.shape), tuple(th.shape)))
        return 0.7 / (1.0 + ((v - th) / (0.4 * th)) ** 2)
    kw = dict(tau_mem=12.0, tau_syn=tau_syn, min_v_mem=-0.5, train_alphas=True, surrogate_grad_fn=custom,
              spike_fn=act.MaxSpike(2), spike_threshold=0.8)
    native, rows = pair(el, el.LIF, **kw)
    g = gen(17)
    xa = (torch.rand(*shape, generator=g) * 4 - 1).cuda().requires_grad_(True)
    xb = xa.detach().clone().requires_grad_(True)
    assert native._use_native_layout(xa) and not rows._use_native_layout(xb)
    w = torch.rand(shape, generator=g).cuda()
    for k in range(2):                                       # the second pass starts from states that carry a graph
        a = native(xa); b = rows(xb)
        assert torch.equal(a, b)
        ((a * w).sum() + native.v_mem.sum()).backward(retain_graph=True)
        ((b * w).sum() + rows.v_mem.sum()).backward(retain_graph=True)
    assert calls and len(calls[0][0]) == 3 and calls[0][1][1] == 1     # (batch, time, neurons), (batch, 1, neurons)
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(native.named_parameters(), rows.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-5 * max(1.0, (shape[0] * shape[1]) ** 0.5))
    assert bool((xa.grad != 0).any())


@pytest.mark.parametrize("tau_syn", [None, 6.0])
@pytest.mark.parametrize("surrogate", ["single_exp", "callable"])
@pytest.mark.parametrize("shape", [(3, 70, 5, 8), (2, 45, 37)])
def test_recorded_states_are_differentiable_on_the_layer_kernels(L, tau_syn, surrogate, shape):
    """``record_states=True`` while training: the records are outputs of the layer Function, and a loss on
    them reaches input and parameters as it does through the (rows, time) Functions
    (reference sinabs/exodus/layers/lif.py:256,290-293)."""
    el, act, _ = L
    kw = dict(tau_mem=12.0, tau_syn=tau_syn, min_v_mem=-0.5, train_alphas=True, record_states=True,
              spike_fn=act.MaxSpike(2), spike_threshold=0.8)
    if surrogate == "callable":
        kw["surrogate_grad_fn"] = lambda v, th: 0.7 / (1.0 + ((v - th) / (0.4 * th)) ** 2)
    native, rows = pair(el, el.LIF, **kw)
    g = gen(23)
    xa = (torch.rand(*shape, generator=g) * 4 - 1).cuda().requires_grad_(True)
    xb = xa.detach().clone().requires_grad_(True)
    assert native._use_native_layout(xa) and not rows._use_native_layout(xb)
    w = [torch.rand(shape, generator=g).cuda() for _ in range(3)]
    def loss(layer, out):
        total = (out * w[0]).sum() + (layer.recordings["v_mem"] * w[1]).sum() + layer.v_mem.sum()
        if tau_syn is not None:
            total = total + (layer.recordings["i_syn"] * w[2]).sum()
        return total
    for k in range(2):
        a = native(xa); b = rows(xb)
        assert torch.equal(a, b)
        assert torch.equal(native.recordings["v_mem"], rows.recordings["v_mem"])
        if tau_syn is not None:
            assert torch.equal(native.recordings["i_syn"], rows.recordings["i_syn"])
        loss(native, a).backward(retain_graph=True); loss(rows, b).backward(retain_graph=True)
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(native.named_parameters(), rows.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-5 * max(1.0, (shape[0] * shape[1]) ** 0.5))
    # a loss on the records alone (no gradient on the spikes at all)
    native.reset_states(); rows.reset_states(); xa.grad = None; xb.grad = None
    native(xa); rows(xb)
    (native.recordings["v_mem"] * w[1]).sum().backward(); (rows.recordings["v_mem"] * w[1]).sum().backward()
    assert_close(xa.grad, xb.grad, "grad input from the records alone")
    assert bool((xa.grad != 0).any())


def test_value_checks_follow_parameter_versions(L, monkeypatch):
    """The range checks wait for the device, so a layer repeats them only after one of its parameters was
    written to; an invalid value is reported at the first call after the write and at every later one."""
    el, act, _ = L
    import sinabs.exodus.layer_function as lf
    import sinabs.exodus.layers.neurons as nm
    calls = []
    real = lf.check_parameters
    def counting(*a, **k):
        calls.append(1)
        return real(*a, **k)
    monkeypatch.setattr(lf, "check_parameters", counting)
    monkeypatch.setattr(nm, "check_parameters", counting)
    layer = el.LIF(tau_mem=10.0, min_v_mem=-1.0, train_alphas=True).cuda()
    x = torch.rand(2, 20, 16, generator=gen(2)).cuda()
    layer(x); layer(x)
    with torch.no_grad():
        layer(x)
    assert len(calls) == 1
    with torch.no_grad():
        layer.alpha_mem.fill_(1.5)
    for _ in range(2):
        with pytest.raises(ValueError):
            layer(x)
    with torch.no_grad():
        with pytest.raises(ValueError):
            layer(x)
    assert len(calls) == 4
    with torch.no_grad():
        layer.alpha_mem.fill_(0.9)
    layer(x); layer(x)
    assert len(calls) == 5
    with torch.no_grad():
        layer.min_v_mem.fill_(3.0)                          # not below the threshold any more
    with pytest.raises(ValueError):
        layer(x)
    with torch.no_grad():
        layer.min_v_mem.fill_(-1.0)
    layer(torch.rand(3, 20, 16, generator=gen(3)).cuda())   # new state shape: checked again
    assert len(calls) == 7


def test_kept_parameter_vectors_follow_writes_to_the_parameters(L):
    """Per-neuron vectors of parameters that are not differentiated are kept between calls; a write to the
    parameter, a replacement or a new state shape must show in the very next call."""
    el, act, _ = L
    x = (torch.rand(2, 40, 24, generator=gen(5)) * 3).cuda()
    def fresh(**kw):
        layer = el.LIF(**kw).cuda()
        with torch.no_grad():
            return layer(x), layer.v_mem
    layer = el.LIF(tau_mem=10.0, min_v_mem=-1.0, spike_threshold=1.0).cuda()
    with torch.no_grad():
        for _ in range(2):
            layer.reset_states(); a = layer(x)
        want, _ = fresh(tau_mem=10.0, min_v_mem=-1.0, spike_threshold=1.0)
        assert torch.equal(a, want)
        layer.spike_threshold.fill_(0.5)                      # in-place write
        layer.reset_states(); a = layer(x)
        want, _ = fresh(tau_mem=10.0, min_v_mem=-1.0, spike_threshold=0.5)
        assert torch.equal(a, want)
        layer.tau_mem.fill_(4.0)
        layer.reset_states(); a = layer(x)
        want, _ = fresh(tau_mem=4.0, min_v_mem=-1.0, spike_threshold=0.5)
        assert torch.equal(a, want)
        layer.min_v_mem = torch.nn.Parameter(torch.tensor(-0.2).cuda(), requires_grad=False)   # replacement
        layer.reset_states(); a = layer(x)
        want, _ = fresh(tau_mem=4.0, min_v_mem=-0.2, spike_threshold=0.5)
        assert torch.equal(a, want)
        b = layer(x[:1])                                       # other state shape
        other = el.LIF(tau_mem=4.0, min_v_mem=-0.2, spike_threshold=0.5).cuda()
        assert torch.equal(b, other(x[:1]))
    # with gradients the decay factor is rebuilt from the time constant in every call
    layer = el.LIF(tau_mem=10.0).cuda()
    assert layer.tau_mem.requires_grad
    layer(x).sum().backward()
    g1 = layer.tau_mem.grad.clone(); layer.tau_mem.grad = None
    layer.reset_states(); layer(x).sum().backward()
    assert torch.equal(layer.tau_mem.grad, g1) and bool(g1.abs() > 0)
