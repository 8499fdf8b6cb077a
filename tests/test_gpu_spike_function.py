"""The experimental spike-generation pair (reference sinabs/exodus/spike.py:7-104,
cuda/experimental_kernels.h) through the C ABI, against the CPU oracle's literal O(T^2) restatement.

The kernels accumulate the pending corrections in one running value instead of subtracting each
spike's tail separately, so potentials are compared within the fp32 tolerance and spike rasters may
differ only where a potential sits within rounding distance of a multiple of the threshold."""
import pytest
import torch

from _util import assert_close, gen, spike_tie_report
from oracle import exodus_ref as ref

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (3, 7), (64, 100), (130, 333), (257, 64), (5, 1000), (1000, 31)]


@pytest.fixture(scope="module")
def hip():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip
    return _hip


def potential(seed, n, t, alpha):
    """A leaky integral of noisy input: what the function is meant to receive."""
    x = torch.randn(n, t, generator=gen(seed)) * 0.5 + 0.15
    return ref.leaky_forward(x.contiguous(), torch.zeros(n), torch.full((n,), alpha))


@pytest.mark.parametrize("n,t", SHAPES)
@pytest.mark.parametrize("alpha", [1.0, 0.9])
@pytest.mark.parametrize("lo,cap", [(None, -1), (-0.4, -1), (-0.4, 2), (None, 1)])
def test_forward_against_oracle(hip, n, t, alpha, lo, cap):
    u = potential(n * 7 + t, n, t, alpha)
    want_v = u.clone()
    want_s = ref.spike_forward(want_v, alpha, 0.8, 1.0, 0.0 if lo is None else lo, lo is not None, cap)
    got_v = u.cuda()
    got_s = hip.spikeForward(got_v, alpha, 0.8, 1.0, 0.0 if lo is None else lo, lo is not None, cap)
    tie_frac, bad = spike_tie_report(got_s, want_s, want_v, torch.ones(n), ulps=64)
    assert bad == 0, f"{bad} rows differ away from a threshold tie"
    same = (got_s.cpu() == want_s).all(1)
    assert same.float().mean() > 0.9 or n < 20
    # the corrected potential is the difference of the raw potential and the accumulated resets, so
    # both sides carry rounding noise of the raw magnitude: the absolute tolerance scales with it
    slack = 1e-5 * u.abs().amax(1, keepdim=True).clamp(min=1.0) + 1e-4 * want_v.abs()
    excess = ((got_v.cpu() - want_v).abs() / slack)[same]
    assert excess.numel() == 0 or excess.max() <= 1.0, f"corrected potential: {excess.max():.3g} x tolerance"
    if cap > 0:
        assert got_s.max() <= cap
    assert (got_s == got_s.round()).all() and (got_s >= 0).all()


def test_forward_bit_exact_on_dyadic_grid(hip):
    """alpha = 1/2 and inputs on a 1/64 grid make every operation exact, so the running-sum form
    must reproduce the oracle bit for bit, lower bound and cap included."""
    n, t = 300, 9
    x = (torch.randint(-96, 192, (n, t), generator=gen(3)).float() / 64.0).contiguous()
    u = ref.leaky_forward(x, torch.zeros(n), torch.full((n,), 0.5))
    for lo, cap in ((None, -1), (-0.5, 2)):
        want_v = u.clone()
        want_s = ref.spike_forward(want_v, 0.5, 0.75, 1.0, 0.0 if lo is None else lo, lo is not None, cap)
        got_v = u.cuda()
        got_s = hip.spikeForward(got_v, 0.5, 0.75, 1.0, 0.0 if lo is None else lo, lo is not None, cap)
        assert torch.equal(got_s.cpu(), want_s) and torch.equal(got_v.cpu(), want_v)
        assert want_s.sum() > 100


@pytest.mark.parametrize("n,t", SHAPES)
@pytest.mark.parametrize("alpha", [1.0, 0.85])
def test_backward_against_oracle(hip, n, t, alpha):
    g = gen(n + 13 * t)
    surr = (torch.rand(n, t, generator=g) * 0.9).contiguous()
    go = torch.randn(n, t, generator=g)
    nc = (torch.rand(n, t, generator=g) > 0.2).float()
    want = ref.spike_backward(surr, go, nc, alpha, 0.7)
    got = hip.spikeBackward(surr.cuda(), go.cuda(), nc.cuda(), alpha, 0.7)
    assert_close(got, want, "grad wrt potential", atol=1e-5 * max(1.0, want.abs().max().item()))


def test_function_end_to_end(hip):
    from sinabs.exodus.spike import SpikeFunction
    from sinabs.exodus._compat import activation as act
    n, t, alpha, c, th, lo = 40, 120, 0.9, 0.8, 1.0, -0.3
    u0 = potential(99, n, t, alpha)
    u = u0.cuda().requires_grad_(True)
    surrogate = act.SingleExponential()
    spikes, v = SpikeFunction.apply(u, c, alpha, surrogate, th, lo, 2)
    assert v.data_ptr() == u.data_ptr()                       # corrected in place, as in the reference
    want_v = u0.clone()
    want_s = ref.spike_forward(want_v, alpha, c, th, lo, True, 2)
    _, bad = spike_tie_report(spikes, want_s, want_v, torch.ones(n), ulps=64)
    assert bad == 0 and spikes.sum() > 0
    w = torch.rand(n, t, generator=gen(5))
    (spikes * w.cuda()).sum().backward()
    vv = v.detach().cpu()
    surr = ref.SingleExponential()(vv, th)
    want_g = ref.spike_backward(surr.contiguous(), w, (vv > lo).float(), alpha, c)
    assert_close(u.grad, want_g, "SpikeFunction grad", atol=1e-5 * max(1.0, want_g.abs().max().item()))


def test_function_argument_errors(hip):
    from sinabs.exodus.spike import SpikeFunction
    from sinabs.exodus._compat import activation as act
    sg = act.SingleExponential()
    u = torch.rand(4, 10).cuda()
    with pytest.raises(ValueError):
        SpikeFunction.apply(u.t(), 1.0, 0.9, sg, 1.0)
    with pytest.raises(ValueError):
        SpikeFunction.apply(u[0], 1.0, 0.9, sg, 1.0)
    with pytest.raises(ValueError):
        SpikeFunction.apply(u, 1.0, 0.9, sg, 1.0, 1.5)
    x = u.clone().requires_grad_(True)
    s, v = SpikeFunction.apply(x, 1.0, 0.9, sg, 0.5)
    with pytest.raises(NotImplementedError):
        (s.sum() + v.sum()).backward()
    empty = hip.spikeForward(torch.empty(0, 5).cuda(), 0.9, 1.0, 1.0, 0.0, False, -1)
    assert empty.shape == (0, 5)
