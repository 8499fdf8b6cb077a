"""A whole forward + backward pass of a small spiking network recorded into a HIP graph
(``torch.cuda.CUDAGraph``) and replayed: every entry point only enqueues kernels on the stream it is
given, so the recording holds the hand-written kernels themselves and a replay skips the host side.

Each replay is compared with the same step run eagerly; between replays the program does ordinary eager
work and waits for the device, so that a node that only works on the first replay is caught."""
import warnings

import pytest
import torch
import torch.nn as nn

from _util import assert_close, gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def el():
    assert torch.cuda.is_available()
    import sinabs.exodus.layers as layers
    return layers


def small_network(el, tau_syn):
    from sinabs.exodus._compat import activation as act
    return nn.Sequential(
        nn.Linear(24, 96, bias=False),
        el.LIF(tau_mem=15.0, tau_syn=tau_syn, min_v_mem=-1.0, spike_fn=act.MaxSpike(2), train_alphas=True, norm_input=False),
        nn.Linear(96, 10, bias=False),
        el.IAF(),
    ).cuda()


def step(model, x, weight):
    """One training-style pass from zero states; returns output spikes, leaves gradients in ``.grad``."""
    for m in model:
        if hasattr(m, "reset_states"):
            m.reset_states()
    out = model(x)
    (out * weight).sum().backward()
    return out


@pytest.mark.parametrize("tau_syn", [None, 4.0])
def test_replays_equal_eager_steps(el, tau_syn):
    torch.manual_seed(11)
    recorded = small_network(el, tau_syn); eager = small_network(el, tau_syn)
    with torch.no_grad():
        recorded[0].weight.mul_(6.0); recorded[2].weight.mul_(4.0)
    eager.load_state_dict(recorded.state_dict())
    batch, steps = 4, 50
    inputs = [(torch.rand(batch, steps, 24, generator=gen(40 + k)) * (1.0 + 0.5 * k)).cuda() for k in range(4)]
    weight = torch.rand(batch, steps, 10, generator=gen(39)).cuda()
    x_static = inputs[0].clone()

    # The usual recipe: a few eager passes on a side stream, gradients released, then the capture -- on the
    # same stream.  Two things keep autograd's per-parameter gradient accumulators from being bound to another
    # stream than the one that is captured (PyTorch warns about such a mismatch, and with the default stream on
    # the other side it makes the engine wait on a stream outside the capture, which ends the capture with an
    # error): (1) the capture runs on the warm-up's stream; (2) the layers' states, which carry the autograd
    # graph of the last warm-up pass and with it every accumulator that pass created, are detached first
    # (``layer.zero_grad()`` does that), so the capture creates its own.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(recorded, x_static, weight)
            recorded.zero_grad(set_to_none=True)
        for m in recorded:
            if hasattr(m, "reset_states"):
                m.zero_grad()                                  # detaches v_mem / i_syn from the warm-up's graph
    torch.cuda.current_stream().wait_stream(side)

    # the recording zeroes and reads the state tensors that exist now; the layers replace them by new ones
    # during the pass, so the program has to keep these alive for as long as it replays the graph
    held = [buf for buf in recorded.buffers()]
    graph = torch.cuda.CUDAGraph()
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        with torch.cuda.graph(graph, stream=side):
            out_static = step(recorded, x_static, weight)
    stream_warnings = [str(w.message) for w in caught if "AccumulateGrad" in str(w.message)]
    assert not stream_warnings, stream_warnings
    grads_static = {k: p.grad for k, p in recorded.named_parameters() if p.grad is not None}
    assert {"0.weight", "1.alpha_mem", "2.weight"} <= set(grads_static)

    active = 0
    for k in (1, 2, 0, 3, 1):
        eager.zero_grad(set_to_none=True)
        want = step(eager, inputs[k], weight)
        torch.cuda.synchronize()
        x_static.copy_(inputs[k])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, want), f"spikes differ on replay with input {k}"
        assert torch.equal(recorded[1].v_mem, eager[1].v_mem) and torch.equal(recorded[3].v_mem, eager[3].v_mem)
        for name, p in eager.named_parameters():
            if p.grad is not None:
                assert_close(grads_static[name], p.grad, f"grad {name}, input {k}", rtol=1e-5, atol=1e-6)
        active += int(want.sum().item() > 0)
    assert active == 5


def test_kernels_run_on_the_current_stream(el):
    """The entry points enqueue on the stream they are handed: work issued under a side stream is
    ordered after that stream's earlier work (here a slow fill that the input depends on) and is not
    visible to the default stream until the streams are joined."""
    layer = el.LIF(tau_mem=10.0, tau_syn=4.0).cuda()
    ref_layer = el.LIF(tau_mem=10.0, tau_syn=4.0).cuda()
    base = (torch.rand(4, 60, 512, generator=gen(21)) * 3).cuda()
    want = ref_layer(base * 2.0)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        x = base.clone()
        for _ in range(50):                                   # a chain of dependent kernels on the side stream
            x = x * 1.0
        x = x * 2.0
        got = layer(x)
    side.synchronize()
    assert torch.equal(got, want)
    assert torch.equal(layer.v_mem, ref_layer.v_mem)


def test_graphed_step_helper_with_placement_enabled(el):
    """``sinabs.exodus.graph.GraphedStep`` records the step; ``hbm.enable()`` is active meanwhile.  During the
    capture the wrappers leave allocation to the capture's own memory pool (memory of the striped range handed out
    there would go back to its pool when the Python tensors die, and be given to the next eager request while every
    replay still writes to it).  Between replays the program allocates and writes eagerly in the striped range;
    every replay must still equal the eager step."""
    import gc
    from sinabs.exodus import hbm
    from sinabs.exodus.graph import GraphedStep
    torch.manual_seed(12)
    recorded = small_network(el, 4.0); eager = small_network(el, 4.0)
    with torch.no_grad():
        recorded[0].weight.mul_(6.0); recorded[2].weight.mul_(4.0)
    eager.load_state_dict(recorded.state_dict())
    batch, steps = 64, 400                                     # the first layer's output is 9.8 MB: a placed tensor
    inputs = [(torch.rand(batch, steps, 24, generator=gen(50 + k)) * (1.0 + 0.5 * k)).cuda() for k in range(3)]
    weight = torch.rand(batch, steps, 10, generator=gen(49)).cuda()
    x_static = inputs[0].clone()
    regions = hbm.enable(gib_striped=6.0)
    try:
        # eagerly the layer's output is placed.  (This pass runs on the default stream and leaves its autograd graph
        # -- and the gradient accumulators of the parameters, bound to that stream -- in the layer's states and firing
        # rate; GraphedStep cuts those loose before it warms up on its own stream.)
        probe = recorded[1](recorded[0](x_static))
        assert regions.pool_of(probe) == hbm.STRIPED
        del probe
        graphed = GraphedStep(recorded, lambda: step(recorded, x_static, weight))
        assert regions.pool_of(graphed.output) is None         # inside the capture: the graph's own pool
        scribbles = []
        for k in (1, 2, 0, 1):
            eager.zero_grad(set_to_none=True)
            want = step(eager, inputs[k], weight)
            # eager work in the striped range, of the sizes the recorded step uses: memory that the recording had
            # taken from there and given back would be handed out here, and the next replay would write into it
            for shape in ((batch, steps, 96), (4, 1024, 1024), (batch, 13, 96)):
                scribbles.append(hbm.empty(shape, weight).fill_(float("nan")))
            torch.cuda.synchronize()
            x_static.copy_(inputs[k])
            got = graphed.replay()
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"spikes differ on replay with input {k}"
            assert torch.equal(recorded[1].v_mem, eager[1].v_mem) and torch.equal(recorded[3].v_mem, eager[3].v_mem)
            for name, p in eager.named_parameters():
                if p.grad is not None:
                    assert_close(dict(recorded.named_parameters())[name].grad, p.grad, f"grad {name}, input {k}",
                                 rtol=1e-5, atol=1e-6)
            assert want.sum().item() > 0
            assert all(bool(torch.isnan(t).all()) for t in scribbles), "a replay wrote into memory of the striped range"
    finally:
        scribbles = graphed = want = got = None
        del eager, recorded
        gc.collect()
        assert hbm.disable() is True
