"""The backward kernel that gives every chunk of 32 steps a lane of its own (layers with few neurons and many steps;
``exodus_layer_backward_time_split`` of include/exodus_hip.h) against the kernel that walks the whole sequence in one lane,
which is itself checked against the CPU oracle (test_gpu_native_layout.py, test_gpu_layer_sweep.py): same gradients within
rtol 1e-4 / atol 1e-5 (the sums associate differently, so not bit for bit), decay-factor gradients under the scaled
criterion of the other tests; and, through the layer API, against autograd through the oracle's step-loop layer.  The
reference has one thread per row in every kernel (reference cuda/lif_kernels.h:296-311)."""
import pytest
import torch

from _util import assert_close, gen

pytestmark = pytest.mark.gpu


@pytest.fixture()
def hip():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip
    before = _hip.backwardTimeSplit(-1)
    yield _hip
    _hip.backwardTimeSplit(before)


def per_neuron(n, seed, lo, hi):
    return (torch.rand(n, generator=gen(seed)) * (hi - lo) + lo).cuda()


@pytest.mark.parametrize("shape,cap,kind,clamp,norm,uniform", [
    ((8, 100, 256), -1, 1, False, False, True),      # the small IAF configuration: 4 chunks, the last of 4 steps
    ((8, 100, 256), -1, 1, False, False, False),
    ((3, 33, 70), 2, 1, True, True, False),          # 2 chunks, the second of one step; neurons do not fill a wave
    ((2, 64, 64), 1, 2, True, True, False),          # whole chunks only
    ((1, 512, 130), 3, 3, True, False, False),       # 16 chunks: the most the kernel takes
    ((64, 300, 10), 1, 1, False, True, True),        # the output layer of the convolutional configuration
    ((2, 257, 1), 2, 1, True, True, False),          # one neuron
    ((5, 96, 200), -1, 3, False, True, False),
    ((4, 128, 20000), 2, 1, True, True, False)])     # 80 000 neurons: 1252 blocks
def test_split_backward_equals_sequential_backward(hip, shape, cap, kind, clamp, norm, uniform):
    b, t, m = shape
    n = b * m
    x = (torch.randn(b, t, m, generator=gen(1)) * 1.2 + 0.6).cuda()
    go = torch.full((1,), 0.7, device="cuda") if uniform else torch.randn(b, t, m, generator=gen(2)).cuda()
    a_mem = per_neuron(n, 3, 0.6, 1.0)
    v0, gv = per_neuron(n, 4, -0.3, 0.5), per_neuron(n, 5, -1.0, 1.0)
    theta, c = per_neuron(n, 6, 0.6, 1.3), per_neuron(n, 7, 0.4, 1.0)
    lo = per_neuron(n, 8, -1.0, -0.1) if clamp else None
    f = hip.layerLifForward(x, v0, None, a_mem, None, c, theta, lo, clamp, cap, True, norm)
    assert f["spikes"].sum().item() > 0
    p0 = {1: 0.5, 2: 0.5, 3: 0.7}[kind]
    args = (go, gv, None, x, f["ckpt_v"], None, v0, None, a_mem, None, c, theta, lo, clamp, cap, True, norm, kind, p0, 1.0)
    hip.backwardTimeSplit(0)
    want = hip.layerLifBackward(*args, gradUniform=uniform)
    hip.backwardTimeSplit(2)
    got = hip.layerLifBackward(*args, gradUniform=uniform)
    again = hip.layerLifBackward(*args, gradUniform=uniform)
    assert all(torch.equal(p, q) for p, q in zip(got, again) if p is not None)       # deterministic
    what = f"{shape} cap {cap} kind {kind}"
    assert not torch.equal(got[0], want[0]) or t <= 32, "the split kernel did not run"
    assert_close(got[0], want[0], f"grad_x, {what}")
    assert_close(got[3], want[3], f"grad v_init, {what}")
    assert_close(got[1], want[1], f"grad alpha_mem, {what}", rtol=1e-4, atol=1e-5 * t ** 0.5 * max(1.0, float(want[1].abs().max()) ** 0.5))
    assert got[2] is None and got[4] is None
    # without checkpoints from the caller (the library's own array) the same kernel runs
    hip.backwardTimeSplit(2)
    own = hip.layerLifBackward(go, gv, None, x, None, None, *args[6:], gradUniform=uniform)
    assert all(torch.equal(p, q) for p, q in zip(own, got) if p is not None)


def test_what_the_split_kernel_does_not_take_runs_on_the_sequential_one(hip):
    """Synapse, a surrogate read from a tensor, more than 16 chunks, a single chunk: mode 2 changes nothing."""
    b, t, m = 2, 70, 96
    n = b * m
    x = (torch.randn(b, t, m, generator=gen(11)) * 1.2 + 0.6).cuda()
    go = torch.randn(b, t, m, generator=gen(12)).cuda()
    a_mem, a_syn = per_neuron(n, 13, 0.6, 1.0), per_neuron(n, 14, 0.4, 0.9)
    zero, one = torch.zeros(n, device="cuda"), torch.ones(n, device="cuda")

    def both(run):
        hip.backwardTimeSplit(0)
        a = run()
        hip.backwardTimeSplit(2)
        b_ = run()
        assert all(torch.equal(p, q) for p, q in zip(a, b_) if p is not None)

    f = hip.layerLifForward(x, zero, zero, a_mem, a_syn, one, one, None, False, 2, True, True)
    both(lambda: hip.layerLifBackward(go, None, None, x, f["ckpt_v"], f["ckpt_i"], zero, zero, a_mem, a_syn, one, one, None,
                                      False, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0))
    f = hip.layerLifForward(x, zero, None, a_mem, None, one, one, None, False, 2, True, True)
    surr = torch.rand(b, t, m, generator=gen(16)).cuda()
    both(lambda: hip.layerLifBackward(go, None, None, x, f["ckpt_v"], None, zero, None, a_mem, None, one, one, None, False, 2,
                                      True, True, hip.SURR_TENSOR, 0.0, 0.0, surr=surr))
    xl = (torch.randn(1, 520, 64, generator=gen(15)) * 1.2 + 0.6).cuda()           # 17 chunks
    fl = hip.layerLifForward(xl, zero[:64], None, a_mem[:64], None, one[:64], one[:64], None, False, 2, True, True)
    both(lambda: hip.layerLifBackward(torch.ones_like(xl), None, None, xl, fl["ckpt_v"], None, zero[:64], None, a_mem[:64],
                                      None, one[:64], one[:64], None, False, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0))
    xs = xl[:, :32].contiguous()                                                      # one chunk
    fs = hip.layerLifForward(xs, zero[:64], None, a_mem[:64], None, one[:64], one[:64], None, False, 2, True, True)
    both(lambda: hip.layerLifBackward(torch.ones_like(xs), None, None, xs, fs["ckpt_v"], None, zero[:64], None, a_mem[:64],
                                      None, one[:64], one[:64], None, False, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0))
    assert hip.backwardTimeSplit(7) == 2 and hip.backwardTimeSplit(-1) == 2           # other values change nothing


@pytest.mark.parametrize("layer_kind", ["iaf", "lif"])
def test_small_layers_against_the_step_loop_layers(hip, layer_kind):
    """A layer small enough for the default mode to split its backward, two chained calls, against autograd through
    the oracle's per-step layer."""
    import sinabs.exodus.layers as el
    from oracle import sinabs_layers as sl
    from sinabs.exodus._compat import activation as act
    assert hip.backwardTimeSplit(-1) == 1
    if layer_kind == "iaf":
        fast, plain = el.IAF(min_v_mem=-0.8).cuda(), sl.IAF(min_v_mem=-0.8).cuda()
    else:
        kw = dict(tau_mem=torch.full((24,), 12.0), spike_fn=act.MaxSpike(2), train_alphas=True, norm_input=True)
        fast, plain = el.LIF(**kw).cuda(), sl.LIF(**kw).cuda()
    # (a neuron without leak never forgets: the rounding of the surrogate's exponential -- hardware exp2 here, torch.exp
    # in the step loop -- adds up along the sequence in BOTH backward kernels alike, 1.6 x the tolerance after 2 x 150
    # steps with either; so the comparison with the step loop uses 2 x 64 steps for IAF, and the two kernels are compared
    # with each other at every length in the test above)
    steps = 64 if layer_kind == "iaf" else 150
    data = (torch.rand(2, 4, steps, 24, generator=gen(21)) * (0.5 if layer_kind == "iaf" else 6.0)).cuda()
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    w = torch.rand(4, steps, 24, generator=gen(22)).cuda()
    for k in range(2):
        a = fast(xa[k]); b_ = plain(xb[k])
        assert torch.equal(a, b_)
    assert a.sum() > 0
    (a * w).sum().backward(); (b_ * w).sum().backward()
    assert_close(xa.grad, xb.grad, "grad input over two chained calls")
    for (k, p), (_, q) in zip(fast.named_parameters(), plain.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-4)
