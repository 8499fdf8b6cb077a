"""Seeded sweep through the layer API: the layer-layout kernels against the (rows, time) Functions on random
layer types, shapes (remainders of the 16- and 32-step stages, widths that do and do not fill memory lines),
options, spike mechanisms, surrogate gradients (the three the kernels know and a callable), state records in
the loss, chained calls whose states carry a graph.

Spikes have to be bit-identical.  Gradients are compared within rtol 1e-4 / atol 1e-5 plus 1e-5 of the tensor's
largest magnitude (per-neuron sums cancel, and the two paths add in different orders).  The subtract value never
exceeds the threshold, which keeps |alpha (1 - c * surrogate)| <= 1: beyond that the backward recurrence grows
exponentially and amplifies rounding differences of either path without bound."""
import random

import pytest
import torch

from _util import gen, note_scaled

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["one lane per neuron", "small layers split over time"])
def backward_kernel_choice(request):
    """Every test of this file runs twice: with the backward kernel that walks a neuron's sequence in one lane only, and
    with the default choice, which hands small layers to the kernel that gives every 32 steps a lane."""
    from sinabs.exodus import _hip
    before = _hip.backwardTimeSplit(0 if request.param.startswith("one") else 1)
    yield
    _hip.backwardTimeSplit(before)


def excess(got, want, rtol=1e-4, atol=1e-5, of_max=1e-5):
    if not got.numel():
        return 0.0
    got, want = got.detach(), want.detach()
    return float(((got - want).abs() / (atol + rtol * want.abs() + of_max * want.abs().max())).max())


def test_random_layers_native_equals_rows_path():
    assert torch.cuda.is_available()
    import sinabs.exodus.layers as el
    from sinabs.exodus._compat import activation as act
    rnd = random.Random(2024)
    worst = 0.0
    for case in range(300):
        b = rnd.choice([1, 2, 3, 5, 8])
        t = rnd.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 50, 64, 65, 96, 100, 130, 257])
        m = rnd.choice([1, 2, 3, 5, 6, 31, 32, 33, 64, 100, 128, 250, 255, 256, 257, 258, 260, 512, 514, 1000, 1024, 2050])
        kind = rnd.choice(["lif", "lif", "lif", "iaf", "leak"])
        g = gen(7000 + case)
        if kind == "leak":
            cls = el.ExpLeak
            kw = dict(tau_mem=(5 + 20 * torch.rand(m, generator=g)) if rnd.random() < 0.5 else 12.0,
                      train_alphas=rnd.random() < 0.5, norm_input=rnd.random() < 0.5, decay_early=rnd.random() < 0.5,
                      record_states=rnd.random() < 0.3)
        else:
            spike = rnd.choice([act.MultiSpike, act.SingleSpike, act.MaxSpike(2), act.MaxSpike(3)])
            surrogate = rnd.choice([act.SingleExponential(), act.PeriodicExponential(), act.Heaviside(window=0.7),
                                    lambda v, th: 0.6 / (1.0 + ((v - th) / (0.5 * th)) ** 2)])
            kw = dict(spike_fn=spike, surrogate_grad_fn=surrogate, spike_threshold=rnd.choice([1.0, 0.6, 1.7]),
                      min_v_mem=rnd.choice([None, -0.5, -1.0]), record_states=rnd.random() < 0.3,
                      tau_syn=rnd.choice([None, None, 4.0, 9.0]), decay_early=rnd.random() < 0.5)
            if rnd.random() < 0.3:
                kw["reset_fn"] = act.MembraneSubtract(subtract_value=kw["spike_threshold"] * rnd.choice([0.4, 0.7, 1.0]))
            cls = el.IAF
            if kind == "lif":
                cls = el.LIF
                kw.update(tau_mem=(5 + 20 * torch.rand(m, generator=g)) if rnd.random() < 0.5 else 15.0,
                          train_alphas=rnd.random() < 0.5, norm_input=rnd.random() < 0.5)
        what = f"case {case}: {cls.__name__} b={b} t={t} m={m} " + ", ".join(
            f"{k}={'tensor' if torch.is_tensor(v) else getattr(v, '__name__', v)}" for k, v in kw.items())
        native = cls(**kw).cuda(); rows = cls(**kw).cuda()
        rows.native_layout = False
        scale = 6.0 if kw.get("norm_input", False) else 0.8
        x = torch.randn(b, t, m, generator=g) * scale + 0.3 * scale
        xa = x.cuda().requires_grad_(True); xb = x.cuda().requires_grad_(True)
        w = torch.rand(b, t, m, generator=g).cuda(); w2 = torch.rand(b, t, m, generator=g).cuda()
        for _ in range(rnd.choice([1, 2])):
            a = native(xa); c = rows(xb)
            if kind == "leak":
                assert excess(a, c, 1e-5, 1e-6, 0.0) <= 1, what
            else:
                assert torch.equal(a, c), what
            la = (a * w).sum(); lc = (c * w).sum()
            if kw["record_states"] and rnd.random() < 0.7:
                for name in native.recordings:
                    la = la + (native.recordings[name] * w2).sum(); lc = lc + (rows.recordings[name] * w2).sum()
            if rnd.random() < 0.5:
                la = la + native.v_mem.sum() * 0.3; lc = lc + rows.v_mem.sum() * 0.3
            la.backward(retain_graph=True); lc.backward(retain_graph=True)
        e = excess(xa.grad, xb.grad)
        note_scaled("layer sweep: grad input", xa.grad, xb.grad, 1e-4, 1e-5, e)
        assert e <= 1, f"{what}: grad input {e:.3g} x tolerance"
        worst = max(worst, e)
        for (k, p), (_, q) in zip(native.named_parameters(), rows.named_parameters()):
            assert (p.grad is None) == (q.grad is None), f"{what}: grad {k}"
            if q.grad is not None:
                e = excess(p.grad, q.grad, atol=1e-5 * max(1.0, (b * t) ** 0.5))
                note_scaled(f"layer sweep: grad {k}", p.grad, q.grad, 1e-4, 1e-5 * max(1.0, (b * t) ** 0.5), e)
                assert e <= 1, f"{what}: grad {k} {e:.3g} x tolerance"
                worst = max(worst, e)
        assert excess(native.v_mem, rows.v_mem, 1e-5, 1e-6, 0.0) <= 1, what
    print(f"largest gradient difference: {worst:.3g} x tolerance")
