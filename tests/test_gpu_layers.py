"""Layer-level parity on the GPU, restating reference tests/test_lif.py, tests/test_iaf.py and
tests/test_exp_leak.py with the oracle's plain step-loop layers (oracle/sinabs_layers.py) in the
role of ``sinabs.layers``.  The step-loop layers are ordinary torch modules; in the model tests
they run on the same device as the EXODUS layers so that the Linear layers in between produce
identical inputs for both, exactly as in the reference's tests."""
from itertools import product

import pytest
import torch
import torch.nn as nn

from _util import assert_close, gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    assert torch.cuda.is_available()
    import sinabs.exodus.layers as el
    from oracle import sinabs_layers as sl
    from sinabs.exodus._compat import activation as act
    return el, sl, act


def correlation_and_scale(a, b):
    a = a.flatten().double(); b = b.flatten().double()
    return (a @ b) / (a.norm() * b.norm() + 1e-30), b.norm() / (a.norm() + 1e-30)


# ------------------------------------------------------------------------------------------ LIF basics
def test_lif_basic(L):
    el, _, _ = L
    tau = torch.tensor(30.0); alpha = torch.exp(-1 / tau)
    x = torch.rand(10, 100, 2, 7, 7, generator=gen(0)).cuda() / (1 - alpha)
    layer = el.LIF(tau_mem=tau).cuda()
    out = layer(x)
    assert layer.does_spike and out.shape == x.shape and not torch.isnan(out).any() and out.sum() > 0
    assert "EXODUS" in repr(layer)
    assert layer.v_mem.shape == (10, 2, 7, 7) and 0 < layer.firing_rate.item()


def test_lif_squeeze(L):
    el, _, _ = L
    tau = torch.tensor(30.0); alpha = torch.exp(-1 / tau)
    x = torch.rand(10 * 100, 2, 7, 7, generator=gen(1)).cuda() / (1 - alpha)
    layer = el.LIFSqueeze(tau_mem=tau, batch_size=10).cuda()
    out = layer(x)
    assert out.shape == x.shape and not torch.isnan(out).any() and out.sum() > 0
    # same numbers as the unsqueezed layer on the 5-D view
    ref_out = el.LIF(tau_mem=tau).cuda()(x.reshape(10, 100, 2, 7, 7))
    assert torch.equal(out, ref_out.flatten(0, 1))


def test_min_v_mem(L):
    el, _, _ = L
    tau = torch.tensor(30.0); alpha = torch.exp(-1 / tau)
    x = torch.rand(10, 1, 2, 7, 7, generator=gen(2)).cuda() / -(1 - alpha)
    layer = el.LIF(tau_mem=tau).cuda(); layer(x)
    assert (layer.v_mem < -0.5).any()
    layer = el.LIF(tau_mem=tau, min_v_mem=-0.5).cuda(); layer(x)
    assert not (layer.v_mem < -0.5).any()


def test_state_reset_and_reinit_on_shape_change(L):
    el, _, _ = L
    layer = el.LIF(tau_mem=30.0).cuda()
    layer.reset_states()
    layer(torch.rand(10, 100, 2, 7, 7, generator=gen(3)).cuda() * 30)
    assert (layer.v_mem != 0).any()
    layer.reset_states()
    assert (layer.v_mem == 0).all()
    layer(torch.rand(4, 20, 5, generator=gen(3)).cuda())
    assert layer.v_mem.shape == (4, 5)


@pytest.mark.parametrize("spike", ["multi", "single", "max3"])
def test_layer_equal_output(L, spike):
    el, sl, act = L
    fn = {"multi": act.MultiSpike, "single": act.SingleSpike, "max3": act.MaxSpike(3)}[spike]
    x = torch.rand((10, 100, 20), generator=gen(4)) * 1e2
    # both on the device: exp(-1/tau) is evaluated where the layer lives, and the CPU and GPU exp
    # differ in the last bit
    plain = sl.LIF(tau_mem=20.0, spike_fn=fn).cuda()
    fast = el.LIF(tau_mem=20.0, spike_fn=fn).cuda()
    a = plain(x.cuda()); b = fast(x.cuda())
    assert a.shape == b.shape and a.sum() > 0
    if spike == "max3":
        assert a.max() == 3
    assert torch.equal(a, b)
    assert torch.equal(plain.v_mem, fast.v_mem)


@pytest.mark.parametrize("decay_early,norm_input,train_alphas", list(product((True, False), (True, False), (True, False))))
def test_fused_synaptic_layer_equals_composed_layer(L, decay_early, norm_input, train_alphas):
    """The layer's one-kernel synapse+membrane path and its two-Function path give identical outputs
    and states, and gradients within fp32 tolerance, over two chained calls."""
    el, _, act = L
    kw = dict(tau_mem=torch.full((12,), 15.0), tau_syn=torch.full((12,), 6.0), min_v_mem=-0.8, norm_input=norm_input,
              train_alphas=train_alphas, decay_early=decay_early, spike_fn=act.MaxSpike(2), record_states=True)
    fused = el.LIF(**kw).cuda(); composed = el.LIF(**kw).cuda(); composed.fuse_synapse = False
    data = torch.rand((2, 5, 60, 12), generator=gen(21)).cuda() * (6.0 if norm_input else 0.6)
    xa = data.clone().requires_grad_(True); xb = data.clone().requires_grad_(True)
    for k in range(2):
        a = fused(xa[k]); b = composed(xb[k])
        assert torch.equal(a, b) and torch.equal(fused.v_mem, composed.v_mem) and torch.equal(fused.i_syn, composed.i_syn)
    assert a.sum() > 0
    w = torch.rand(a.shape, generator=gen(22)).cuda()
    ((a * w).sum() + fused.recordings["v_mem"].sum() * 0.1).backward()
    ((b * w).sum() + composed.recordings["v_mem"].sum() * 0.1).backward()
    assert_close(xa.grad, xb.grad, "grad input")
    for (k, p), (_, q) in zip(fused.named_parameters(), composed.named_parameters()):
        if q.grad is not None:
            assert_close(p.grad, q.grad, f"grad {k}", rtol=1e-4, atol=1e-5)


def test_record_states(L):
    el, sl, _ = L
    x = torch.rand((3, 40, 6), generator=gen(5)) * 3
    plain = sl.LIF(tau_mem=10.0, tau_syn=4.0, record_states=True)
    fast = el.LIF(tau_mem=10.0, tau_syn=4.0, record_states=True).cuda()
    a = plain(x); b = fast(x.cuda())
    assert set(fast.recordings) == {"v_mem", "i_syn"} and fast.recordings["v_mem"].shape == x.shape
    assert_close(fast.recordings["i_syn"], plain.recordings["i_syn"], "i_syn recording")
    assert torch.equal(fast.recordings["v_mem"][:, -1], fast.v_mem)


# ------------------------------------------------------------------------------------------ models
def lif_model(layers_mod, tau_mem, tau_leak, n_in, n_out, train_alphas=False, norm_input=True):
    kw = dict(train_alphas=train_alphas, norm_input=norm_input)
    return nn.Sequential(
        nn.Linear(n_in, 16, bias=False), layers_mod.ExpLeak(tau_mem=tau_leak, **kw), layers_mod.LIF(tau_mem=tau_mem, **kw),
        nn.Linear(16, 32, bias=False), layers_mod.ExpLeak(tau_mem=tau_leak, **kw), layers_mod.LIF(tau_mem=tau_mem, **kw),
        nn.Linear(32, n_out, bias=False), layers_mod.ExpLeak(tau_mem=tau_leak, **kw), layers_mod.LIF(tau_mem=tau_mem, **kw),
    )


def copy_linear(src, dst, gain=1.0):
    """Same Linear weights in both models; ``gain`` scales them so that activity reaches the last layer."""
    for i in (0, 3, 6):
        with torch.no_grad():
            src[i].weight.mul_(gain)
        dst[i].load_state_dict(src[i].state_dict())


def test_model_equal_output(L):
    el, sl, _ = L
    torch.manual_seed(0)
    plain = lif_model(sl, 20.0, 10.0, 16, 10).cuda(); fast = lif_model(el, 20.0, 10.0, 16, 10).cuda()
    copy_linear(fast, plain, gain=40.0)
    x = torch.rand((10, 100, 16), generator=gen(6)).cuda() * 1e3
    a = plain(x); b = fast(x)
    assert a.shape == b.shape == (10, 100, 10) and a.sum() > 0
    assert torch.equal(a, b)


@pytest.mark.parametrize("train_alphas,norm_input", list(product((True, False), (True, False))))
def test_state_dict_transfer(L, train_alphas, norm_input):
    """reference tests/test_lif.py:202-249: parameters and states move between the two kinds of model."""
    el, sl, _ = L
    torch.manual_seed(1)
    kw = dict(tau_mem=20.0, tau_leak=10.0, n_in=16, n_out=10, train_alphas=train_alphas, norm_input=norm_input)
    plain = lif_model(sl, **kw).cuda(); fast = lif_model(el, **kw).cuda()
    copy_linear(fast, plain, gain=40.0 if norm_input else 1.0)
    plain.load_state_dict(fast.state_dict())
    x = torch.rand((10, 100, 16), generator=gen(7)).cuda() * (1.0 if norm_input else 5e-2) * 20
    plain(x); fast(x)
    new_plain = lif_model(sl, **kw).cuda(); new_plain(x); new_plain.load_state_dict(fast.state_dict())
    new_fast = lif_model(el, **kw).cuda(); new_fast(x); new_fast.load_state_dict(plain.state_dict())
    outs = [m(x) for m in (plain, fast, new_plain, new_fast)]
    assert outs[0].sum() > 0
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert list(plain.state_dict()) == list(fast.state_dict())


@pytest.mark.parametrize("train_alphas,norm_input,train_time_consts", list(product((True, False), (True, False), (True, False))))
def test_model_compare_grads(L, train_alphas, norm_input, train_time_consts):
    """reference tests/test_lif.py:255-350 (two chained forward calls, then one backward)."""
    el, sl, _ = L
    torch.manual_seed(2)
    kw = dict(tau_mem=20.0, tau_leak=10.0, n_in=2, n_out=2, train_alphas=train_alphas, norm_input=norm_input)
    plain = lif_model(sl, **kw).cuda(); fast = lif_model(el, **kw).cuda()
    if not train_time_consts:
        for m in (plain, fast):
            for n, p in m.named_parameters():
                if "tau" in n or "alpha" in n:
                    p.requires_grad_(False)
    copy_linear(fast, plain)
    data = torch.rand((2, 2, 5, 2), generator=gen(8)).cuda() * (40.0 if norm_input else 2.0)
    for inp in data:
        a = plain(inp)
    nn.functional.mse_loss(a, torch.ones_like(a)).backward()
    for inp in data:
        b = fast(inp)
    nn.functional.mse_loss(b, torch.ones_like(b)).backward()
    assert torch.equal(a, b)
    for lp, lf in zip(plain, fast):
        if hasattr(lp, "v_mem"):
            assert_close(lf.v_mem, lp.v_mem, "layer state", rtol=1e-4, atol=1e-6)
    gp = {k: p.grad for k, p in plain.named_parameters() if p.grad is not None}
    gf = {k: p.grad for k, p in fast.named_parameters() if p.grad is not None}
    assert set(gp) == set(gf)
    for k in gp:
        assert_close(gf[k], gp[k], f"grad {k}", rtol=1e-4, atol=1e-6)
        if gp[k].abs().max() > 0:
            corr, scale = correlation_and_scale(gp[k], gf[k])
            assert (1 - corr) < 1e-5 and abs(scale - 1) < 1e-3


@pytest.mark.parametrize("train_alphas,norm_input,tau_syn,decay_early",
                         [(t, n, s, d) for t, n, s in product((True, False), (True, False), (None, 30.0))
                          for d in ((True, False) if s else (True,))])
def test_single_layer_compare_grads(L, train_alphas, norm_input, tau_syn, decay_early):
    """reference tests/test_lif.py:356-423: per-channel tau, min_v_mem, non-zero initial v_mem and i_syn.
    ``decay_early=False`` has no counterpart in plain sinabs, so it is checked for consistency only
    (fused kernel vs the composed Functions, tests/test_gpu_synaptic.py)."""
    el, sl, _ = L
    n_ch = 16
    kw = dict(tau_mem=torch.ones(n_ch) * 20.0, tau_syn=tau_syn, spike_threshold=1.0, min_v_mem=-1.0,
              norm_input=norm_input, train_alphas=train_alphas, record_states=True)
    plain = sl.LIF(**kw); plain.clip_mode = "max"
    fast = el.LIF(decay_early=decay_early, **kw).cuda()
    g = gen(9)
    x = torch.rand((2, 10, n_ch), generator=g) * (8.0 if norm_input else 1.0)
    v0 = torch.rand(2, n_ch, generator=g); i0 = torch.rand(2, n_ch, generator=g)
    plain.v_mem = v0.clone(); fast.v_mem = v0.clone().cuda()
    if tau_syn is not None:
        plain.i_syn = i0.clone(); fast.i_syn = i0.clone().cuda()
    b = fast(x.cuda()); nn.functional.mse_loss(b, torch.ones_like(b)).backward()
    if not decay_early:
        assert torch.isfinite(b).all()
        assert all(torch.isfinite(p.grad).all() for p in fast.parameters() if p.grad is not None)
        return
    a = plain(x); nn.functional.mse_loss(a, torch.ones_like(a)).backward()
    assert a.sum() == b.sum().cpu()
    gp = {k: p.grad for k, p in plain.named_parameters() if p.grad is not None}
    gf = {k: p.grad.cpu() for k, p in fast.named_parameters() if p.grad is not None}
    assert set(gp) == set(gf) and len(gp) > 0
    for k in gp:
        assert_close(gf[k], gp[k], f"grad {k}", rtol=1e-3, atol=1e-6)
        corr, scale = correlation_and_scale(gp[k], gf[k])
        assert abs(corr - 1) < 1e-5 and abs(scale - 1) < 1e-3


@pytest.mark.parametrize("tau_syn", [None, 30.0])
@pytest.mark.parametrize("train_alphas", [True, False])
def test_loss_on_recorded_states_against_the_step_loop(L, tau_syn, train_alphas):
    """A loss on ``recordings`` (potential after each reset, synaptic current) and on the spikes: gradients of
    the layer kernels against torch autograd through the plain per-step loop (the records are differentiable
    in the reference too, sinabs/exodus/layers/lif.py:256,290-293)."""
    el, sl, _ = L
    n_ch = 12
    kw = dict(tau_mem=torch.linspace(10.0, 30.0, n_ch), tau_syn=tau_syn, spike_threshold=1.0, min_v_mem=-1.0,
              norm_input=True, train_alphas=train_alphas, record_states=True)
    plain = sl.LIF(**kw); plain.clip_mode = "max"
    fast = el.LIF(**kw).cuda()
    g = gen(31)
    x = torch.rand((3, 40, n_ch), generator=g) * 8.0
    w = [torch.rand((3, 40, n_ch), generator=g) for _ in range(3)]
    v0 = torch.rand(3, n_ch, generator=g)
    plain.v_mem = v0.clone(); fast.v_mem = v0.clone().cuda()
    xa = x.clone().requires_grad_(True); xb = x.clone().cuda().requires_grad_(True)
    def loss(layer, out, dev):
        total = (out * w[0].to(dev)).sum() + (layer.recordings["v_mem"] * w[1].to(dev)).sum()
        if tau_syn is not None:
            total = total + (layer.recordings["i_syn"] * w[2].to(dev)).sum()
        return total
    a = plain(xa); loss(plain, a, "cpu").backward()
    b = fast(xb); loss(fast, b, "cuda").backward()
    assert fast._use_native_layout(xb)
    assert torch.equal(a, b.cpu())
    assert_close(fast.recordings["v_mem"].cpu(), plain.recordings["v_mem"], "recorded v_mem")
    assert_close(xb.grad.cpu(), xa.grad, "grad input", rtol=1e-4, atol=1e-5)
    gp = {k: p.grad for k, p in plain.named_parameters() if p.grad is not None}
    gf = {k: p.grad.cpu() for k, p in fast.named_parameters() if p.grad is not None}
    assert set(gp) == set(gf) and len(gp) > 0
    for k in gp:
        assert_close(gf[k], gp[k], f"grad {k}", rtol=1e-3, atol=1e-5)


def test_alpha_grad_trace_per_timestep(L):
    """reference tests/test_lif.py:426-485: d out[t] / d alpha_mem for every t, lower bound 0, synapses."""
    el, sl, _ = L
    kw = dict(tau_mem=torch.ones(1) * 20.0, tau_syn=30.0, spike_threshold=1.2, min_v_mem=0.0, norm_input=False,
              train_alphas=True, record_states=True)
    plain = sl.LIF(**kw); plain.clip_mode = "max"
    fast = el.LIF(**kw).cuda()
    x = torch.zeros((1, 20, 1)); x[:, 1] = 2
    g = gen(10); v0 = torch.rand(1, 1, generator=g); i0 = torch.rand(1, 1, generator=g)

    def trace(model, dev):
        grads = []
        for t in range(20):
            model.zero_grad(); model.reset_states()
            model.v_mem = v0.clone().to(dev); model.i_syn = i0.clone().to(dev)
            out = model(x.to(dev))
            out[0, t, 0].backward()
            grads.append(0.0 if model.alpha_mem.grad is None else model.alpha_mem.grad.item())
        return torch.tensor(grads)

    assert_close(trace(fast, "cuda"), trace(plain, "cpu"), "alpha_mem gradient per time step", rtol=1e-3, atol=1e-7)


# ------------------------------------------------------------------------------------------ IAF
def test_iaf_basic_squeeze_and_minvmem(L):
    el, _, _ = L
    x = torch.rand(10, 100, 2, 7, 7, generator=gen(11)).cuda()
    layer = el.IAF().cuda(); out = layer(x)
    assert out.shape == x.shape and out.sum() > 0 and "EXODUS" in repr(layer)
    sq = el.IAFSqueeze(batch_size=10).cuda()
    assert torch.equal(sq(x.flatten(0, 1)), out.flatten(0, 1))
    neg = -torch.rand(10, 1, 2, 7, 7, generator=gen(12)).cuda()
    a = el.IAF().cuda(); a(neg); assert (a.v_mem < -0.5).any()
    b = el.IAF(min_v_mem=-0.5).cuda(); b(neg); assert not (b.v_mem < -0.5).any()


def test_iaf_equal_output_many_spikes(L):
    el, sl, _ = L
    x = torch.zeros((10, 100, 16)); x[:, :10] = 1e4                       # reference tests/test_iaf.py:71-79
    a = sl.IAF()(x); b = el.IAF().cuda()(x.cuda()).cpu()
    assert (a != 0).any() and torch.equal(a, b)


def iaf_model(layers_mod, n_in=16, n_out=10, min_v_mem=None):
    return nn.Sequential(nn.Linear(n_in, 16, bias=False), layers_mod.IAF(min_v_mem=min_v_mem),
                         nn.Linear(16, 32, bias=False), layers_mod.IAF(min_v_mem=min_v_mem),
                         nn.Linear(32, n_out, bias=False), layers_mod.IAF(min_v_mem=min_v_mem))


@pytest.mark.parametrize("min_v_mem", [None, -1.0])
def test_iaf_model_chained_calls_and_grads(L, min_v_mem):
    """reference tests/test_iaf.py:188-241: three forward calls carrying state, then one backward."""
    el, sl, _ = L
    torch.manual_seed(3)
    plain = iaf_model(sl, min_v_mem=min_v_mem).cuda(); fast = iaf_model(el, min_v_mem=min_v_mem).cuda()
    for m in plain:
        if hasattr(m, "clip_mode"):
            m.clip_mode = "max"
    for i in (0, 2, 4):
        plain[i].load_state_dict(fast[i].state_dict())
    data = torch.rand((3, 10, 100, 16), generator=gen(13)).cuda()
    for inp in data:
        a = plain(inp)
    nn.functional.mse_loss(a, torch.ones_like(a)).backward()
    for inp in data:
        b = fast(inp)
    nn.functional.mse_loss(b, torch.ones_like(b)).backward()
    assert torch.equal(a, b) and a.sum() > 0
    for i in (1, 3, 5):
        assert_close(fast[i].v_mem, plain[i].v_mem, "state", rtol=1e-4, atol=1e-5)
    for (k, p), (_, q) in zip(plain.named_parameters(), fast.named_parameters()):
        if p.grad is not None:
            assert_close(q.grad, p.grad, f"grad {k}", rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------------------------------------ ExpLeak
def test_expleak_basic_decay_early_squeeze(L):
    el, _, _ = L
    x = torch.rand(100, 2, 7, 7, generator=gen(14)).cuda()
    layer = el.ExpLeak(tau_mem=30.0).cuda(); out = layer(x)
    assert not layer.does_spike and out.shape == x.shape and out.sum() > 0 and "EXODUS" in repr(layer)
    dec = el.ExpLeak(tau_mem=30.0, decay_early=True).cuda()(x)
    assert torch.allclose(dec, out * layer.alpha_mem_calculated)
    x4 = torch.rand(10 * 100, 2, 7, 7, generator=gen(15)).cuda()
    sq = el.ExpLeakSqueeze(tau_mem=30.0, batch_size=10).cuda()(x4)
    assert sq.shape == x4.shape and sq.sum() > 0


def test_expleak_membrane_decay_closed_form(L):
    """reference tests/test_exp_leak.py:53-75"""
    el, _, _ = L
    tau = torch.tensor(30.0); alpha = torch.exp(-1 / tau)
    x = torch.zeros(10, 100, 2, 7, 7).cuda(); x[:, 0] = 1 / (1 - alpha)
    layer = el.ExpLeak(tau_mem=tau, norm_input=True, decay_early=False).cuda()
    out = layer(x)
    assert torch.allclose(out[:, 0], torch.tensor(1.0).cuda())
    assert (out[:, -1] == layer.v_mem).all()
    assert torch.isclose(layer.v_mem, (alpha ** 99).cuda(), atol=1e-8).all()


@pytest.mark.parametrize("train_alphas,norm_input", list(product((True, False), (True, False))))
def test_expleak_equal_output_and_grads(L, train_alphas, norm_input):
    el, sl, _ = L
    kw = dict(tau_mem=torch.full((16,), 10.0), train_alphas=train_alphas, norm_input=norm_input)
    plain = sl.ExpLeak(**kw); fast = el.ExpLeak(**kw).cuda()
    x = torch.zeros((10, 100, 16)); x[:, :10] = 1e2 * torch.rand(10, 10, 16, generator=gen(16))
    xa = x.clone().requires_grad_(True); xb = x.clone().cuda().requires_grad_(True)
    a = plain(xa); b = fast(xb)
    assert (a != 0).any() and torch.equal(a, b.cpu())
    w = torch.rand(a.shape, generator=gen(17))
    (a * w).sum().backward(); (b * w.cuda()).sum().backward()
    assert_close(xb.grad, xa.grad, "grad input", rtol=1e-4, atol=1e-5)
    for (k, p), (_, q) in zip(plain.named_parameters(), fast.named_parameters()):
        assert_close(q.grad, p.grad, f"grad {k}", rtol=1e-3, atol=1e-4)


# ------------------------------------------------------------------------------------------ conv SNN
def conv_snn(layers_mod, batch_size):
    """The convolutional configuration of the benchmark description: conv / pooling work on
    (batch*time, C, H, W), the neuron layers are the Squeeze variants in between."""
    return nn.Sequential(
        nn.Conv2d(2, 32, 3), layers_mod.IAFSqueeze(batch_size=batch_size), nn.AvgPool2d(2),
        nn.Conv2d(32, 64, 3), layers_mod.IAFSqueeze(batch_size=batch_size), nn.Flatten(),
        nn.Linear(64 * 14 * 14, 10), layers_mod.IAFSqueeze(batch_size=batch_size),
    )


def test_conv_snn_end_to_end(L):
    el, sl, _ = L
    torch.manual_seed(4)
    batch, steps = 3, 40
    fast = conv_snn(el, batch).cuda(); plain = conv_snn(sl, batch).cuda()
    for i in (0, 3, 6):
        with torch.no_grad():
            fast[i].weight.mul_(3.0)
        plain[i].load_state_dict(fast[i].state_dict())
    x = (torch.rand(batch, steps, 2, 34, 34, generator=gen(30)) < 0.02).float().cuda()
    labels = torch.randint(0, 10, (batch,), generator=gen(31)).cuda()

    def run(model):
        out = model(x.flatten(0, 1)).reshape(batch, steps, 10)
        loss = nn.functional.cross_entropy(out.sum(1), labels)
        loss.backward()
        return out, loss

    out_f, loss_f = run(fast); out_p, loss_p = run(plain)
    assert out_p.sum() > 0 and torch.equal(out_f, out_p)
    assert torch.equal(fast[1].v_mem, plain[1].v_mem)
    assert_close(loss_f, loss_p, "loss", rtol=1e-6, atol=1e-7)
    for (k, p), (_, q) in zip(plain.named_parameters(), fast.named_parameters()):
        if p.grad is not None:
            assert_close(q.grad, p.grad, f"grad {k}", rtol=1e-4, atol=1e-5)
