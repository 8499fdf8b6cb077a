"""The benchmark configurations at their full sizes.  A CPU comparison of 2e9 neuron-timesteps is
out of reach, so these tests check (a) a random sample of neurons against the CPU oracle, bit for bit
in the forward direction and within rtol 1e-4 / atol 1e-5 for gradients, and (b) size-independent
properties: integer spike counts within the cap, the fused spike total, the lower bound, linearity
of the backward pass in the incoming gradient."""
import math

import pytest
import torch

from _util import assert_close, gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    assert torch.cuda.is_available()
    from oracle import exodus_ref as ref
    from sinabs.exodus import _hip as hip
    return hip, ref


def need_gib(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * 2 ** 30:
        pytest.skip(f"needs {gib} GiB of free device memory")


def sample_columns(x, idx_b, idx_m):
    """(B,T,M) device tensor -> (n_sample, T) CPU rows for the sampled (batch, neuron) pairs."""
    return x[idx_b, :, idx_m].contiguous().cpu()


def test_c5_synaptic_lif_full_size(mods):
    hip, ref = mods
    need_gib(60)
    B, T, M = 16, 2000, 65536
    N = B * M
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn(B, T, M, generator=g, device=dev) * 0.5 + 0.05
    am, asyn = math.exp(-1 / 20.0), math.exp(-1 / 5.0)
    full = lambda v: torch.full((N,), v, device=dev)
    a_mem, a_syn, lo, one, zero = full(am), full(asyn), full(-1.0), full(1.0), full(0.0)
    res = hip.layerLifForward(x, zero, zero, a_mem, a_syn, one, one, lo, True, 2, True, True)
    spikes = res["spikes"]

    # properties
    assert float(res["spike_sum"]) == float(spikes.sum(dtype=torch.float64))
    assert bool(((spikes == 0) | (spikes == 1) | (spikes == 2)).all())
    assert float(res["v_last"].min()) >= -1.0 - 2.0                     # post-reset: clamp minus at most 2 resets
    assert 0 < float(res["spike_sum"]) < N * T

    # sampled neurons against the oracle (composition of its pieces, as the reference layer composes them)
    cg = gen(5)
    n_s = 1024
    ib = torch.randint(0, B, (n_s,), generator=cg); im = torch.randint(0, M, (n_s,), generator=cg)
    xs = sample_columns(x, ib.to(dev), im.to(dev))
    r = lambda v: torch.full((n_s,), v)
    i_rows = ref.leaky_forward((xs * r(asyn)[:, None]).contiguous(), r(0.0), r(asyn))
    ws, wv = ref.integrate_and_fire_forward(((1.0 - r(am)[:, None]) * i_rows).contiguous(), r(am), r(0.0), r(1.0), None,
                                            r(-1.0), 2)
    assert torch.equal(sample_columns(spikes, ib.to(dev), im.to(dev)), ws)
    flat = (ib * M + im)
    assert torch.equal(res["v_last"].cpu()[flat], (wv - ws)[:, -1])
    assert torch.equal(res["i_last"].cpu()[flat], i_rows[:, -1])

    # backward: sampled neurons against the oracle's chained backward, and linearity in grad_spikes
    go1 = torch.randn(B, T, M, generator=g, device=dev)
    bw = lambda go: hip.layerLifBackward(go, None, None, x, res["ckpt_v"], res["ckpt_i"], zero, zero, a_mem, a_syn, one,
                                         one, lo, True, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    gi1, gam1, gas1, _, _ = bw(go1)
    gos = sample_columns(go1, ib.to(dev), im.to(dev))
    g_u, g_am_lif, _ = ref.integrate_and_fire_backward(gos, None, wv, ws, r(0.0), r(am), r(1.0), r(1.0), r(-1.0),
                                                       ref.SingleExponential(), True, gate_initial=True)
    g_i = ((1.0 - r(am)[:, None]) * g_u).contiguous()
    g_xin, g_as_leaky, _ = ref.leaky_integrator_backward(g_i, i_rows, r(0.0), r(asyn), True)
    want_gx = g_xin * r(asyn)[:, None]
    assert_close(sample_columns(gi1, ib.to(dev), im.to(dev)), want_gx, "grad_x of sampled neurons")
    want_gam = g_am_lif - (g_u * i_rows).sum(1)
    want_gas = g_as_leaky + (g_xin * xs).sum(1)
    assert_close(gam1.cpu()[flat], want_gam, "grad alpha_mem of sampled neurons", rtol=1e-4, atol=1e-5 * T ** 0.5)
    assert_close(gas1.cpu()[flat], want_gas, "grad alpha_syn of sampled neurons", rtol=1e-4, atol=1e-5 * T ** 0.5)
    del go1
    gi2, _, _, _, _ = bw(gi1 * 0 + 1.0)                                   # grad = ones
    gi3, _, _, _, _ = bw(gi1 * 0 + 3.0)
    assert_close(gi3[:2, :, :4096], 3.0 * gi2[:2, :, :4096], "backward is linear in grad_spikes")


def test_c2_lif_full_size(mods):
    hip, ref = mods
    need_gib(30)
    B, T, M = 32, 300, 128 * 32 * 32
    N = B * M
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(B, T, M, generator=g, device=dev) * 0.3 + 0.1
    am = math.exp(-1 / 20.0)
    full = lambda v: torch.full((N,), v, device=dev)
    a_mem, one, zero = full(am), full(1.0), full(0.0)
    res = hip.layerLifForward(x, zero, None, a_mem, None, one, one, None, False, 1, True, True)
    spikes = res["spikes"]
    assert float(res["spike_sum"]) == float(spikes.sum(dtype=torch.float64))
    assert bool(((spikes == 0) | (spikes == 1)).all())
    cg = gen(6); n_s = 2048
    ib = torch.randint(0, B, (n_s,), generator=cg); im = torch.randint(0, M, (n_s,), generator=cg)
    xs = sample_columns(x, ib.to(dev), im.to(dev))
    r = lambda v: torch.full((n_s,), v)
    ws, wv = ref.integrate_and_fire_forward(((1.0 - r(am)[:, None]) * xs).contiguous(), r(am), r(0.0), r(1.0), None, None, 1)
    assert torch.equal(sample_columns(spikes, ib.to(dev), im.to(dev)), ws)
    go = torch.ones(B, T, M, device=dev)
    gi, gam, _, gv0, _ = hip.layerLifBackward(go, None, None, x, res["ckpt_v"], None, zero, None, a_mem, None, one, one,
                                              None, False, 1, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    g_u, g_am_lif, g_v0 = ref.integrate_and_fire_backward(torch.ones(n_s, T), None, wv, ws, r(0.0), r(am), r(1.0), r(1.0),
                                                          None, ref.SingleExponential(), True, gate_initial=True)
    assert_close(sample_columns(gi, ib.to(dev), im.to(dev)), (1.0 - r(am)[:, None]) * g_u, "grad_x of sampled neurons")
    flat = ib * M + im
    assert_close(gv0.cpu()[flat], g_v0, "grad v_init of sampled neurons")
    assert_close(gam.cpu()[flat], g_am_lif - (g_u * xs).sum(1), "grad alpha of sampled neurons", rtol=1e-4,
                 atol=1e-5 * T ** 0.5)


def test_c5_rows_kernels_full_size_sampled(mods):
    """The (rows, time) kernels at 1 048 576 x 2000 (offsets beyond 2^31): sampled rows against the oracle."""
    hip, ref = mods
    need_gib(45)
    n, t = 1 << 20, 2000
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(7)
    x = torch.randn(n, t, generator=g, device=dev) * 0.5 + 0.05
    alpha = torch.rand(n, generator=g, device=dev); th = torch.rand(n, generator=g, device=dev) + 0.5
    zero = torch.zeros(n, device=dev); lo = -torch.ones(n, device=dev)
    s = torch.empty_like(x); v = torch.empty_like(x)
    hip.lifForward(s, v, x, zero, alpha, th, th, lo, True, 2)
    idx = torch.cat([torch.tensor([0, 1, n - 2, n - 1, (1 << 20) - 64 * 3 - 1]), torch.randint(0, n, (507,), generator=gen(8))])
    c = lambda z: z[idx.to(dev)].contiguous().cpu()
    ws, wv = ref.lif_forward(c(x), c(zero), c(alpha), c(th), c(th), c(lo), True, 2)
    assert torch.equal(c(s), ws) and torch.equal(c(v), wv)
    go = torch.randn(n, t, generator=g, device=dev)
    gi, ga, ginit = hip.lifBackwardFused(go, None, v, zero, alpha, th, th, lo, True, 2, hip.SURR_SINGLE_EXP, 0.5, 1.0,
                                         needAlphaGrad=True)
    wgi, wga, wginit = ref.integrate_and_fire_backward(c(go), None, wv, ws, c(zero), c(alpha), c(th), c(th), c(lo),
                                                       ref.SingleExponential(), True, gate_initial=True)
    assert_close(c(gi), wgi, "grad_input of sampled rows")
    assert_close(c(ginit), wginit, "grad_init of sampled rows")
    assert_close(c(ga), wga, "grad_alpha of sampled rows", rtol=1e-4, atol=1e-5 * t ** 0.5)


def test_layer_kernels_index_tensors_beyond_2_31_elements(mods):
    """(9, 2000, 131072) has 2.36e9 elements per tensor, more than a 32-bit index holds.  Neurons are
    independent, so the last batch element computed inside the big call must equal the same batch
    element computed alone, bit for bit, forward and backward, spiking and leaky."""
    hip, _ = mods
    need_gib(80)
    B, T, M = 9, 2000, 131072
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(12)
    x = torch.randn(B, T, M, generator=g, device=dev) * 0.5 + 0.05
    go = torch.randn(B, T, M, generator=g, device=dev)
    full = lambda n, v: torch.full((n,), v, device=dev)
    am, asn = math.exp(-1 / 20.0), math.exp(-1 / 5.0)

    def spiking(xx, gg):
        n = xx.shape[0] * M
        f = hip.layerLifForward(xx, full(n, 0.0), full(n, 0.0), full(n, am), full(n, asn), full(n, 1.0), full(n, 1.0),
                                full(n, -1.0), True, 2, True, True)
        b = hip.layerLifBackward(gg, None, None, xx, f["ckpt_v"], f["ckpt_i"], full(n, 0.0), full(n, 0.0), full(n, am),
                                 full(n, asn), full(n, 1.0), full(n, 1.0), full(n, -1.0), True, 2, True, True,
                                 hip.SURR_SINGLE_EXP, 0.5, 1.0)
        return f["spikes"], f["v_last"], b[0], b[1]

    s_big, v_big, gx_big, ga_big = spiking(x, go)
    s_one, v_one, gx_one, ga_one = spiking(x[B - 1:].contiguous(), go[B - 1:].contiguous())
    assert torch.equal(s_big[B - 1], s_one[0]) and s_one.sum() > 0
    assert torch.equal(v_big[(B - 1) * M:], v_one)
    assert torch.equal(gx_big[B - 1], gx_one[0]) and torch.equal(ga_big[(B - 1) * M:], ga_one)
    del s_big, gx_big, s_one, gx_one

    def leaky(xx, gg):
        n = xx.shape[0] * M
        out, v_last = hip.layerLeakyForward(xx, full(n, 0.0), full(n, am), True, True)
        gi, ga, _ = hip.layerLeakyBackward(gg, None, out, xx, full(n, 0.0), full(n, am), True, True, True)
        return out, gi, ga

    o_big, gi_big, ga_big = leaky(x, go)
    o_one, gi_one, ga_one = leaky(x[B - 1:].contiguous(), go[B - 1:].contiguous())
    assert torch.equal(o_big[B - 1], o_one[0]) and torch.equal(gi_big[B - 1], gi_one[0])
    assert torch.equal(ga_big[(B - 1) * M:], ga_one)


def test_identical_batch_elements_give_identical_results_at_full_size(mods):
    """Every element of the outputs is checked here, not a sample: all 16 batch elements of a C5-sized
    input are copies of one another, neurons are independent, so every output must repeat 16 times bit
    for bit -- on the layer kernels and on the (rows, time) kernels, forward and backward.  A write that
    goes astray anywhere in 2e9 elements breaks the repetition."""
    hip, _ = mods
    need_gib(90)
    B, T, M = 16, 2000, 65536
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(21)
    x = (torch.randn(1, T, M, generator=g, device=dev) * 0.5 + 0.05).expand(B, T, M).contiguous()
    go = torch.randn(1, T, M, generator=g, device=dev).expand(B, T, M).contiguous()
    n = B * M
    full = lambda v: torch.full((n,), v, device=dev)
    am, asn = math.exp(-1 / 20.0), math.exp(-1 / 5.0)

    def repeats(z):
        z = z.reshape(B, -1)
        return bool((z == z[:1]).all())

    f = hip.layerLifForward(x, full(0.0), full(0.0), full(am), full(asn), full(1.0), full(1.0), full(-1.0), True, 2,
                            True, True)
    assert f["spikes"].sum() > 0
    assert repeats(f["spikes"]) and repeats(f["v_last"]) and repeats(f["i_last"]) and repeats(f["ckpt_v"])
    b = hip.layerLifBackward(go, None, None, x, f["ckpt_v"], f["ckpt_i"], full(0.0), full(0.0), full(am), full(asn),
                             full(1.0), full(1.0), full(-1.0), True, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    assert all(repeats(t) for t in b if t is not None)
    del f, b

    out, v_last = hip.layerLeakyForward(x, full(0.0), full(am), True, True)
    gi, ga, gv = hip.layerLeakyBackward(go, None, out, x, full(0.0), full(am), True, True, True)
    gi2 = hip.layerLeakyBackward(go, None, None, None, None, full(am), False, False, False)[0]
    assert repeats(out) and repeats(v_last) and repeats(gi) and repeats(ga) and repeats(gv) and repeats(gi2)
    del out, gi, gi2

    # (rows, time): row r = b * M + m, so rows repeat with period M
    xr = x.movedim(1, 2).reshape(n, T).contiguous(); gor = go.movedim(1, 2).reshape(n, T).contiguous()
    del x, go
    s = torch.empty_like(xr); v = torch.empty_like(xr)
    hip.lifForward(s, v, xr, full(0.0), full(am), full(1.0), full(1.0), full(-1.0), True, 2)
    assert repeats(s) and repeats(v)
    gir, gar, ginit = hip.lifBackwardFused(gor, None, v, full(0.0), full(am), full(1.0), full(1.0), full(-1.0), True, 2,
                                           hip.SURR_SINGLE_EXP, 0.5, 1.0, needAlphaGrad=True)
    assert repeats(gir) and repeats(gar) and repeats(ginit)


def test_c3_expleak_full_size(mods):
    """ExpLeak with one trainable decay factor per channel, tau ~ U[5, 50], input ~ N(0, 1), at
    (64, 1000, 4096) (the reference's counterpart at small size: tests/test_exp_leak.py:100-136).
    The output and the input gradient of 768 sampled (batch, channel) rows and the batch-summed
    per-channel alpha gradient of 48 whole channels against the oracle's restatement of the reference
    kernels; both input options of the layer, weighted output gradients."""
    hip, ref = mods
    from _util import note_scaled, worst
    need_gib(8)
    B, T, M = 64, 1000, 4096
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn(B, T, M, generator=g, device=dev)
    go = torch.randn(B, T, M, generator=g, device=dev)
    tau = 5.0 + 45.0 * torch.rand(M, generator=g, device=dev)
    alpha_c = torch.exp(-1.0 / tau)                               # (M,)
    alpha = alpha_c.expand(B, M).flatten().contiguous()
    v0 = torch.randn(B * M, generator=g, device=dev) * 0.2
    cg = gen(9)
    ib = torch.randint(0, B, (768,), generator=cg); im = torch.randint(0, M, (768,), generator=cg)
    chans = torch.randperm(M, generator=cg)[:48]
    for decay_early, norm_input in ((False, False), (True, True)):
        out, v_last = hip.layerLeakyForward(x, v0, alpha, decay_early, norm_input)
        gi, ga, gv0 = hip.layerLeakyBackward(go, None, out, x, v0, alpha, decay_early, norm_input, True)

        def oracle(xs, gos, a, v0s):
            """rows through the oracle: scaled input -> leaky forward -> backward, chain rule for the scalings"""
            k = (1.0 - a) if norm_input else torch.ones_like(a)
            xin = k[:, None] * xs
            if decay_early:
                xin = xin * a[:, None]
            o = ref.leaky_forward(xin.contiguous(), v0s, a)
            g_in, g_a, g_v0 = ref.leaky_integrator_backward(gos.contiguous(), o, v0s, a, True)
            gx = g_in * k[:, None] * (a[:, None] if decay_early else 1.0)
            # d xin / d alpha = -x (norm) * (alpha if decay) + k x (decay)
            dxin = torch.zeros_like(xs)
            if norm_input:
                dxin = dxin - xs * (a[:, None] if decay_early else 1.0)
            if decay_early:
                dxin = dxin + k[:, None] * xs
            g_a = g_a + (g_in.double() * dxin.double()).sum(1).float()
            # natural size of the alpha gradient's rounding error: it is a sum over time of products
            # g_t * (out_{t-1} + d xin_t / d alpha) with both signs, whose terms are far from 1 here (outputs
            # and adjoints of a slow integrator driven by N(0, 1) reach +-10), so the absolute tolerance
            # scales with the root of the sum of squared terms (= sqrt(T) for terms of size 1)
            prev = torch.cat([v0s[:, None], o[:, :-1]], 1)
            spread = ((g_in.double() * (prev.double() + dxin.double())) ** 2).sum(1).sqrt().float()
            return o, gx, g_a, g_v0, spread

        # sampled rows
        a_s = alpha_c.cpu()[im]; flat = ib * M + im
        o, gx, g_a, g_v0, spread = oracle(sample_columns(x, ib.to(dev), im.to(dev)),
                                          sample_columns(go, ib.to(dev), im.to(dev)), a_s, v0.cpu()[flat])
        got_o = sample_columns(out, ib.to(dev), im.to(dev))
        if not (decay_early or norm_input):
            assert torch.equal(got_o, o)                              # same operations in the same order
        assert_close(got_o, o, "output of sampled rows")
        assert torch.equal(v_last.cpu()[flat], got_o[:, -1])
        assert_close(sample_columns(gi, ib.to(dev), im.to(dev)), gx, "grad_x of sampled rows")
        assert_close(gv0.cpu()[flat], g_v0, "grad v_init of sampled rows")
        print(f"per-row alpha grad of sampled rows: {worst(ga.cpu()[flat], g_a)}")
        note_scaled("C3 per-row alpha gradient (atol 1e-5 x root of the summed squared terms)", ga.cpu()[flat], g_a, 1e-4,
                    float(1e-5 * spread.max()))
        err = (ga.cpu()[flat].double() - g_a.double()).abs() / (1e-5 * spread.clamp(min=1.0) + 1e-4 * g_a.abs()).double()
        assert float(err.max()) <= 1.0, f"grad alpha of sampled rows: {float(err.max()):.3g} x tolerance"
        # whole channels: the per-channel gradient is the sum over the batch (what autograd's expand does)
        xs = x[:, :, chans.to(dev)].permute(2, 0, 1).reshape(-1, T).cpu()      # (48 * B, T), channel-major
        gos = go[:, :, chans.to(dev)].permute(2, 0, 1).reshape(-1, T).cpu()
        a_rows = alpha_c.cpu()[chans].repeat_interleave(B)
        v0_rows = v0.view(B, M)[:, chans.to(dev)].T.reshape(-1).cpu()
        _, _, g_a, _, spread = oracle(xs, gos, a_rows, v0_rows)
        want = g_a.double().view(48, B).sum(1)
        spread = (spread.double().view(48, B) ** 2).sum(1).sqrt()
        got = ga.view(B, M).double().sum(0).cpu()[chans]
        print(f"per-channel alpha grad: {worst(got, want)}")
        note_scaled("C3 per-channel alpha gradient (atol 1e-5 x root of the summed squared terms)", got, want, 1e-4,
                    float(1e-5 * spread.max()))
        err = (got - want).abs() / (1e-5 * spread.clamp(min=1.0) + 1e-4 * want.abs())
        assert float(err.max()) <= 1.0, f"per-channel alpha gradient: {float(err.max()):.3g} x tolerance"


def test_c1_iaf_full_shape():
    """The smallest configuration exactly as described: IAF layer, input (8, 100, 256) ~ U[0, 0.5],
    threshold 1, membrane subtract, SingleExponential surrogate, loss = sum of spikes -- the whole
    tensor against the CPU step loop with autograd, and against the closed form floor(cumsum(x))."""
    import sinabs.exodus.layers as el
    from oracle import sinabs_layers as sl
    x = torch.rand(8, 100, 256, generator=gen(0)) * 0.5
    fast = el.IAF().cuda(); plain = sl.IAF()
    xa = x.clone().requires_grad_(True); xb = x.clone().cuda().requires_grad_(True)
    a = plain(xa); b = fast(xb)
    assert torch.equal(b.cpu(), a) and a.sum() > 0
    # integrate-and-fire identity for non-negative input: spikes up to t = floor(cumsum(x) / theta)
    steps = torch.cumsum(x.double(), 1)
    total = b.detach().cpu().double().cumsum(1)
    assert float((total - steps.floor()).abs().max().item()) <= 1.0          # fp32 sums vs fp64: ties at most one step apart
    assert torch.equal(b.cpu().sum(1), a.sum(1))
    assert torch.equal(fast.v_mem.cpu(), plain.v_mem)
    a.sum().backward(); b.sum().backward()
    assert bool((xa.grad != 0).any())
    assert_close(xb.grad, xa.grad, "grad input")


def test_c4_conv_snn_full_shape():
    """The convolutional configuration at its full shape (batch 64, 300 steps, 2 x 34 x 34 Bernoulli(0.02)
    input, cross-entropy on spike counts): this package's layers against plain step-loop layers with
    autograd, both on the GPU with identical weights -- spikes of all three neuron layers bit for bit,
    loss and weight gradients within tolerance."""
    import torch.nn as nn
    import sinabs.exodus.layers as el
    from oracle import sinabs_layers as sl
    need_gib(120)
    batch, steps = 64, 300

    def net(mod):
        return nn.Sequential(
            nn.Conv2d(2, 32, 3), mod.IAFSqueeze(batch_size=batch), nn.AvgPool2d(2),
            nn.Conv2d(32, 64, 3), mod.IAFSqueeze(batch_size=batch), nn.Flatten(),
            nn.Linear(64 * 14 * 14, 10), mod.IAFSqueeze(batch_size=batch))

    torch.manual_seed(4)
    fast = net(el).cuda(); plain = net(sl).cuda()
    for i in (0, 3, 6):
        with torch.no_grad():
            fast[i].weight.mul_(3.0)
        plain[i].load_state_dict(fast[i].state_dict())
    x = (torch.rand(batch, steps, 2, 34, 34, generator=gen(30)) < 0.02).float().cuda()
    labels = torch.randint(0, 10, (batch,), generator=gen(31)).cuda()
    taps = {}

    def run(model, name):
        hooks = [model[i].register_forward_hook(lambda m, a, o, i=i: taps.__setitem__((name, i), o.detach()))
                 for i in (1, 4, 7)]
        out = model(x.flatten(0, 1)).reshape(batch, steps, 10)
        loss = nn.functional.cross_entropy(out.sum(1), labels)
        loss.backward()
        for h in hooks:
            h.remove()
        return out, loss

    out_f, loss_f = run(fast, "fast")
    out_p, loss_p = run(plain, "plain")
    for i in (1, 4, 7):
        assert taps[("plain", i)].sum() > 0 and torch.equal(taps[("fast", i)], taps[("plain", i)]), f"spikes of layer {i}"
    assert torch.equal(fast[1].v_mem, plain[1].v_mem) and torch.equal(fast[4].v_mem, plain[4].v_mem)
    assert_close(loss_f, loss_p, "loss", rtol=1e-6, atol=1e-7)
    from _util import worst
    for (k, p), (_, q) in zip(plain.named_parameters(), fast.named_parameters()):
        if p.grad is not None:
            print(f"grad {k}: {worst(q.grad, p.grad)}")
            # sums over 64 x 300 x positions of products: judged relative to the gradient's own scale
            assert_close(q.grad, p.grad, f"grad {k}", rtol=1e-4, atol=1e-5 * max(1.0, float(p.grad.abs().max())))
