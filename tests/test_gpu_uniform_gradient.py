"""One value as the gradient of every output element -- the loss ``out.sum()`` of the reference's own tests
(reference tests/test_spike_functions.py:50, tests/test_leak_functions.py:22), which autograd hands to a backward
pass as a scalar expanded with strides of zero (``out.mean()`` does not: torch divides the expansion and hands over
an ordinary tensor).  The layer kernels take the scalar
itself (``grad_spikes_uniform`` / ``grad_out_uniform`` of include/exodus_hip.h) and read one tensor less.

Checked: the kernel instances against the ordinary ones on a written-out constant gradient (bit for bit: the
arithmetic is the same), and the layers under a ``sum()`` loss against the step-loop layers of the oracle with
autograd (rtol 1e-4 / atol 1e-5, spikes equal)."""
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
def hip():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip
    return _hip


def per_neuron(n, seed, lo, hi):
    return (torch.rand(n, generator=gen(seed)) * (hi - lo) + lo).cuda()


@pytest.mark.parametrize("shape,syn,cap,kind", [
    ((3, 70, 96), True, 2, 1), ((2, 64, 512), False, 1, 1), ((1, 33, 130), True, -1, 2), ((4, 5, 64), False, 3, 3),
    ((2, 100, 1), True, 1, 3), ((1, 1, 7), False, 2, 1), ((2, 257, 48), True, 2, 2)])
def test_spiking_backward_with_one_gradient_value_equals_the_dense_call(hip, shape, syn, cap, kind):
    b, t, m = shape
    n = b * m
    x = (torch.randn(b, t, m, generator=gen(1)) * 2.0 + 1.5).cuda()
    a_mem, a_syn = per_neuron(n, 2, 0.7, 0.99), per_neuron(n, 3, 0.5, 0.95) if syn else None
    v0, i0 = per_neuron(n, 4, -0.2, 0.4), per_neuron(n, 5, -0.1, 0.3) if syn else None
    theta, c, lo = per_neuron(n, 6, 0.6, 1.2), per_neuron(n, 7, 0.5, 1.0), per_neuron(n, 8, -0.9, -0.2)
    gv, gi = per_neuron(n, 9, -1.0, 1.0), per_neuron(n, 10, -1.0, 1.0) if syn else None
    f = hip.layerLifForward(x, v0, i0, a_mem, a_syn, c, theta, lo, True, cap, True, True)
    assert f["spikes"].sum().item() > 0 or t * n < 64
    p0 = {1: 0.5, 2: 0.5, 3: 0.7}[kind]
    for value in (1.0, -0.37):
        one = torch.full((1,), value, device="cuda")
        dense = torch.full((b, t, m), value, device="cuda")
        args = (gv, gi, x, f["ckpt_v"], f["ckpt_i"], v0, i0, a_mem, a_syn, c, theta, lo, True, cap, True, True, kind, p0, 1.0)
        want = hip.layerLifBackward(dense, *args)
        got = hip.layerLifBackward(one, *args, gradUniform=True)
        for k, (g, w) in enumerate(zip(got, want)):
            assert (g is None) == (w is None)
            if g is not None:
                assert torch.equal(g, w), f"output {k} differs for gradient value {value}"
        # ... and through the entry point that keeps its checkpoints in the library's own memory
        again = hip.layerLifBackward(one, gv, gi, x, None, None, *args[5:], gradUniform=True)
        assert all(torch.equal(g, w) for g, w in zip(again, want) if g is not None)
    with pytest.raises(RuntimeError):
        hip.layerLifBackward(one, gv, gi, x, f["ckpt_v"], f["ckpt_i"], v0, i0, a_mem, a_syn, c, theta, lo, True, cap,
                             True, True, hip.SURR_TENSOR, 0.5, 1.0, surr=torch.ones_like(x), gradUniform=True)
    with pytest.raises(RuntimeError):
        hip.layerLifBackward(dense, *args, gradUniform=True)      # a whole tensor is not one value


@pytest.mark.parametrize("shape,decay_early,norm_input,alpha_grad", [
    ((3, 70, 96), False, False, True), ((2, 64, 512), True, True, True), ((1, 33, 130), False, True, False),
    ((4, 5, 64), True, False, True), ((2, 100, 1), False, False, True), ((2, 257, 48), True, True, False)])
def test_leaky_backward_with_one_gradient_value_equals_the_dense_call(hip, shape, decay_early, norm_input, alpha_grad):
    b, t, m = shape
    n = b * m
    x = torch.randn(b, t, m, generator=gen(11)).cuda()
    alpha, v0, gv = per_neuron(n, 12, 0.6, 0.99), per_neuron(n, 13, -0.5, 0.5), per_neuron(n, 14, -1.0, 1.0)
    out, _ = hip.layerLeakyForward(x, v0, alpha, decay_early, norm_input)
    for value in (1.0, 0.013):
        one = torch.full((1,), value, device="cuda")
        dense = torch.full((b, t, m), value, device="cuda")
        want = hip.layerLeakyBackward(dense, gv, out, x, v0, alpha, decay_early, norm_input, alpha_grad)
        got = hip.layerLeakyBackward(one, gv, out, x, v0, alpha, decay_early, norm_input, alpha_grad, shape=shape)
        for k, (g, w) in enumerate(zip(got, want)):
            assert (g is None) == (w is None)
            if g is not None:
                assert torch.equal(g, w), f"output {k} differs for gradient value {value}"


@pytest.mark.parametrize("loss,tau_syn,squeeze", list(product(("sum", "scaled sum", "sum+rate"), (None, 4.0), (False, True))))
def test_layers_under_a_sum_loss_against_the_step_loop_layers(loss, tau_syn, squeeze):
    """``out.sum().backward()`` (and a multiple of the sum, and a sum plus the layer's firing rate, whose gradient
    is a second scalar) through the layer: the gradient arrives as a broadcast scalar, the kernel gets the scalar, and the
    results agree with autograd through the oracle's per-step layer."""
    import sinabs.exodus.layers as el
    from oracle import sinabs_layers as sl
    from sinabs.exodus._compat import activation as act
    from sinabs.exodus import layer_function
    kw = dict(tau_mem=15.0, tau_syn=tau_syn, min_v_mem=-0.7, spike_fn=act.MaxSpike(2), train_alphas=True)
    fast = (el.LIFSqueeze(batch_size=3, **kw) if squeeze else el.LIF(**kw)).cuda()
    plain = (sl.LIFSqueeze(batch_size=3, **kw) if squeeze else sl.LIF(**kw)).cuda()
    data = (torch.rand(3, 90, 4, 10, generator=gen(31)) * (5.0 if tau_syn is None else 2.0)).cuda()
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    seen = []
    original = layer_function._hip.layerLifBackward

    def spy(*a, **k):
        seen.append((tuple(a[0].shape), bool(k.get("gradUniform"))))
        return original(*a, **k)

    layer_function._hip.layerLifBackward = spy
    try:
        a = fast(xa.flatten(0, 1) if squeeze else xa)
        la = {"sum": a.sum(), "scaled sum": a.sum() * 0.07, "sum+rate": a.sum() + 50.0 * fast.firing_rate}[loss]
        la.backward()
    finally:
        layer_function._hip.layerLifBackward = original
    assert seen == [((1,), True)], seen                        # the kernel was handed one value, not a tensor
    b = plain(xb.flatten(0, 1) if squeeze else xb)
    lb = {"sum": b.sum(), "scaled sum": b.sum() * 0.07, "sum+rate": b.sum() + 50.0 * plain.firing_rate}[loss]
    lb.backward()
    assert torch.equal(a, b) and a.sum().item() > 0
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(fast.named_parameters(), plain.named_parameters()):
        assert (p.grad is None) == (q.grad is None), k
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("train_alphas,norm_input", [(True, False), (True, True), (False, False)])
def test_leaky_layer_under_a_sum_loss_against_the_step_loop_layer(train_alphas, norm_input):
    import sinabs.exodus.layers as el
    from oracle import sinabs_layers as sl
    from sinabs.exodus import layer_function
    tau = 5.0 + 45.0 * torch.rand(24, generator=gen(41))
    kw = dict(tau_mem=tau, train_alphas=train_alphas, norm_input=norm_input)
    fast, plain = el.ExpLeak(**kw).cuda(), sl.ExpLeak(**kw).cuda()
    data = torch.randn(5, 130, 24, generator=gen(42)).cuda()
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    seen = []
    original = layer_function._hip.layerLeakyBackward

    def spy(*a, **k):
        seen.append((tuple(a[0].shape), k.get("shape")))
        return original(*a, **k)

    layer_function._hip.layerLeakyBackward = spy
    try:
        a = fast(xa)
        a.sum().backward()
    finally:
        layer_function._hip.layerLeakyBackward = original
    assert seen == [((1,), (5, 130, 24))], seen
    b = plain(xb)
    b.sum().backward()
    assert_close(a, b, "output")
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(fast.named_parameters(), plain.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-5 * 130 ** 0.5)
