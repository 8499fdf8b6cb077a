"""Parity of every C-ABI entry point with the CPU oracle, on the GPU, through ctypes.

Forward results are compared bit for bit (same operations in the same order, no fused
multiply-add on either side).  Backward results use the linear-time reverse recurrence where
the oracle sums the reference's quadratic form, so they are compared within the stated fp32
tolerance rtol 1e-4 / atol 1e-5.
"""
import pytest
import torch

from _util import ATOL, RTOL, assert_close, assert_close_rowscaled, gen, lif_case

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (2, 10), (63, 31), (64, 32), (65, 33), (70, 100), (129, 37), (257, 64), (300, 301), (1000, 300)]


@pytest.fixture(scope="module")
def hip():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from sinabs.exodus import _hip
    return _hip


@pytest.fixture(scope="module")
def ref():
    from oracle import exodus_ref
    return exodus_ref


def D(x):
    return None if x is None else x.cuda()


@pytest.mark.parametrize("n,t", SHAPES)
def test_leaky_forward_bitwise(hip, ref, n, t):
    g = gen(n * 1000 + t)
    x = torch.randn(n, t, generator=g); v0 = torch.randn(n, generator=g); a = torch.rand(n, generator=g)
    out = hip.leakyForward(D(x), D(v0), D(a))
    assert torch.equal(out.cpu(), ref.leaky_forward(x, v0, a))


@pytest.mark.parametrize("n,t", SHAPES)
def test_leaky_backward_entry_points(hip, ref, n, t):
    g = gen(n * 1000 + t + 1)
    x = torch.randn(n, t, generator=g); v0 = torch.randn(n, generator=g); a = torch.rand(n, generator=g)
    go = torch.randn(n, t, generator=g)
    out = ref.leaky_forward(x, v0, a)
    want_gi = ref.leaky_backward(go, a)
    want_ga = ref.leaky_backward_alpha(go, out, v0, a)
    assert torch.equal(hip.leakyBackward(D(go), D(a)).cpu(), want_gi)
    # alpha gradient: sum over up to t products per row, reference accumulates in fp32
    assert_close(hip.leakyBackwardAlpha(D(go), D(out), D(v0), D(a)), want_ga, "leakyBackwardAlpha",
                 rtol=RTOL, atol=ATOL * max(1.0, t ** 0.5))
    gi, ga, ginit = hip.leakyBackwardFused(D(go), D(a), output=D(out), vmemInitial=D(v0), needAlphaGrad=True)
    assert torch.equal(gi.cpu(), want_gi)
    assert torch.equal(ginit.cpu(), a * want_gi[:, 0])
    assert_close(ga, want_ga, "fused alpha grad", rtol=RTOL, atol=ATOL * max(1.0, t ** 0.5))
    gi2, ga2, ginit2 = hip.leakyBackwardFused(D(go), D(a))
    assert ga2 is None and torch.equal(gi2.cpu(), want_gi) and torch.equal(ginit2.cpu(), a * want_gi[:, 0])


@pytest.mark.parametrize("n,t", SHAPES)
@pytest.mark.parametrize("cap", [-1, 1, 2])
@pytest.mark.parametrize("use_lo", [False, True])
def test_lif_forward_bitwise(hip, ref, n, t, cap, use_lo):
    c = lif_case(n * 1000 + t + 2, n, t, lo=use_lo)
    s = torch.empty(n, t, device="cuda"); v = torch.empty(n, t, device="cuda")
    hip.lifForward(s, v, D(c["x"]), D(c["v0"]), D(c["alpha"]), D(c["c"]), D(c["theta"]), D(c["lo"]), use_lo, cap)
    ws, wv = ref.lif_forward(c["x"], c["v0"], c["alpha"], c["c"], c["theta"], c["lo"], use_lo, cap)
    assert torch.equal(v.cpu(), wv)
    assert torch.equal(s.cpu(), ws)


@pytest.mark.parametrize("cap", [-1, 0, 1, 2, 3])
def test_lif_forward_other_caps_and_nonpositive_thresholds(hip, ref, cap):
    """Caps beyond the usual ones and thresholds that are zero or negative (the count then comes from
    the quotient, converted to unsigned with saturation as the device does): still bit for bit."""
    n, t = 130, 77
    c = lif_case(900 + cap, n, t, lo=True, scale=1.5, shift=0.4)
    th = c["theta"].clone()
    th[::3] = -0.2 * th[::3]
    th[1::7] = 0.0
    s = torch.empty(n, t, device="cuda"); v = torch.empty(n, t, device="cuda")
    hip.lifForward(s, v, D(c["x"]), D(c["v0"]), D(c["alpha"]), D(c["c"]), D(th), D(c["lo"]), True, cap)
    ws, wv = ref.lif_forward(c["x"], c["v0"], c["alpha"], c["c"], th, c["lo"], True, cap)
    assert torch.equal(s.cpu(), ws) and torch.equal(v.cpu(), wv)
    assert ws[2::3].max() >= min(3, cap if cap >= 0 else 3) or cap == 0


def test_lif_forward_many_spikes_per_step(hip, ref):
    # the regime of reference tests/test_iaf.py:71-79 and tests/test_lif.py:78: inputs of 1e2..1e4 thresholds
    n, t = 40, 50
    g = gen(5)
    x = torch.rand(n, t, generator=g) * 1e4
    one = torch.ones(n)
    s = torch.empty(n, t, device="cuda"); v = torch.empty(n, t, device="cuda")
    hip.lifForward(s, v, D(x), D(torch.zeros(n)), D(one * 0.95), D(one), D(one), None, False, -1)
    ws, wv = ref.lif_forward(x, torch.zeros(n), one * 0.95, one, one, None, False, -1)
    assert torch.equal(s.cpu(), ws) and torch.equal(v.cpu(), wv) and ws.max() > 255


@pytest.mark.parametrize("n,t", SHAPES)
def test_lif_backward_tensor_entry_points(hip, ref, n, t):
    g = gen(n * 1000 + t + 3)
    surr = torch.rand(n, t, generator=g); gg = torch.randn(n, t, generator=g)
    nc = (torch.rand(n, t, generator=g) > 0.2).float()
    a = torch.rand(n, generator=g); c = 0.2 + torch.rand(n, generator=g)
    vpost = torch.randn(n, t, generator=g); v0 = torch.randn(n, generator=g)
    csub = (a * c).contiguous()
    assert_close(hip.lifBackward(D(surr), D(gg), D(nc), D(a), D(csub)), ref.lif_backward(surr, gg, nc, a, csub),
                 "lifBackward")
    tol = dict(rtol=RTOL, atol=ATOL * max(1.0, t ** 0.5))
    for gate in (False, True):
        got = hip.lifBackwardAlpha(D(surr), D(gg), D(vpost), D(v0), D(nc), D(a), D(c), gateInitial=gate)
        want = ref.lif_backward_alpha(surr, gg, vpost, v0, nc, a, c, gate_initial=gate)
        assert_close(got, want, f"lifBackwardAlpha gate={gate}", **tol)


# parameters chosen so that |alpha (1 - c s)| stays <= 1 for the random rows of lif_case (c <= 0.8,
# theta >= 0.5): the gradient recurrence is then contractive and the element-wise tolerance applies
SURROGATES = [("single", 1, 0.5, 1.0), ("single", 1, 0.7, 0.6), ("periodic", 2, 0.5, 1.0), ("periodic", 2, 0.25, 0.7),
              ("heaviside", 3, 0.5, 0.0), ("heaviside", 3, 1.0, 0.0)]


def _surrogate(ref, name, p0, p1):
    if name == "single":
        return ref.SingleExponential(p0, p1)
    if name == "periodic":
        return ref.PeriodicExponential(p0, p1)
    return ref.Heaviside(p0)


@pytest.mark.parametrize("n,t", [(2, 10), (65, 33), (70, 100), (300, 301), (1000, 300)])
@pytest.mark.parametrize("name,kind,p0,p1", SURROGATES)
@pytest.mark.parametrize("cap,use_lo,use_gv", [(-1, False, False), (2, True, True), (1, True, False), (-1, False, True)])
def test_lif_backward_fused(hip, ref, n, t, name, kind, p0, p1, cap, use_lo, use_gv):
    c = lif_case(n * 1000 + t + 4, n, t, lo=use_lo)
    fn = _surrogate(ref, name, p0, p1)
    ws, wv = ref.lif_forward(c["x"], c["v0"], c["alpha"], c["c"], c["theta"], c["lo"], use_lo, cap)
    gv = c["gv"] if use_gv else None
    want_gi, want_ga, want_ginit = ref.integrate_and_fire_backward(
        c["go"], gv, wv, ws, c["v0"], c["alpha"], c["c"], c["theta"], c["lo"], fn, True, gate_initial=True)
    tol_a = dict(rtol=RTOL, atol=ATOL * max(1.0, t ** 0.5))
    # in-kernel surrogate
    gi, ga, ginit = hip.lifBackwardFused(D(c["go"]), D(gv), D(wv), D(c["v0"]), D(c["alpha"]), D(c["c"]), D(c["theta"]),
                                         D(c["lo"]), use_lo, cap, kind, p0, p1, needAlphaGrad=True)
    assert_close(gi, want_gi, "grad_input")
    assert_close(ginit, want_ginit, "grad_init")
    assert_close(ga, want_ga, "grad_alpha", **tol_a)
    # the same kernel fed with a surrogate tensor (path taken by arbitrary callables)
    surr = fn(wv, c["theta"].unsqueeze(1)).contiguous()
    gi2, ga2, ginit2 = hip.lifBackwardFused(D(c["go"]), D(gv), D(wv), D(c["v0"]), D(c["alpha"]), D(c["c"]),
                                            D(c["theta"]), D(c["lo"]), use_lo, cap, hip.SURR_TENSOR, surr=D(surr),
                                            needAlphaGrad=True)
    assert_close(gi2, want_gi, "grad_input (tensor surrogate)")
    assert_close(ginit2, want_ginit, "grad_init (tensor surrogate)")
    assert_close(ga2, want_ga, "grad_alpha (tensor surrogate)", **tol_a)
    # without alpha gradient the other two outputs are unchanged
    gi3, ga3, ginit3 = hip.lifBackwardFused(D(c["go"]), D(gv), D(wv), None, D(c["alpha"]), D(c["c"]), D(c["theta"]),
                                            D(c["lo"]), use_lo, cap, kind, p0, p1)
    assert ga3 is None and torch.equal(gi3, gi) and torch.equal(ginit3, ginit)


def test_lif_backward_fused_expanding_recurrence(hip, ref):
    """A sharp, tall surrogate (width 0.3, scale 2) makes |alpha (1 - c s)| reach ~8: gradients grow
    to 1e5 along a row and fp32 rounding is amplified alike in the reference's quadratic sum and in
    the reverse recurrence.  Both are then accurate relative to the row's magnitude, which is what
    is asserted; the float64 recurrence is the yardstick."""
    n, t = 1000, 300
    c = lif_case(n * 1000 + t + 4, n, t, lo=False)
    fn = ref.SingleExponential(0.3, 2.0)
    ws, wv = ref.lif_forward(c["x"], c["v0"], c["alpha"], c["c"], c["theta"], None, False, -1)
    surr = fn(wv, c["theta"].unsqueeze(1))
    gi64, ga64, _ = ref.lif_backward_recurrence_f64(surr, surr * c["go"], torch.ones_like(surr), c["alpha"], c["c"],
                                                    wv - c["c"].unsqueeze(1) * ws, c["v0"])
    want_gi, _, _ = ref.integrate_and_fire_backward(c["go"], None, wv, ws, c["v0"], c["alpha"], c["c"], c["theta"],
                                                    None, fn, False)
    gi, ga, _ = hip.lifBackwardFused(D(c["go"]), None, D(wv), D(c["v0"]), D(c["alpha"]), D(c["c"]), D(c["theta"]),
                                     None, False, -1, 1, 0.3, 2.0, needAlphaGrad=True)
    assert_close_rowscaled(want_gi, gi64, "reference quadratic sum vs float64")
    assert_close_rowscaled(gi, gi64, "HIP reverse recurrence vs float64")
    assert_close_rowscaled(ga, ga64, "HIP alpha gradient vs float64", atol=ATOL * t ** 0.5)


def test_unaligned_pointers_take_the_scalar_path(hip, ref):
    # a view starting 4 bytes into an allocation is not 16-byte aligned
    n, t = 70, 64
    g = gen(9)
    buf = torch.randn(n * t + 1, generator=g)
    x = buf[1:].view(n, t)
    v0 = torch.randn(n, generator=g); a = torch.rand(n, generator=g)
    xd = buf.cuda()[1:].view(n, t)
    assert xd.data_ptr() % 16 != 0 and xd.is_contiguous()
    assert torch.equal(hip.leakyForward(xd, D(v0), D(a)).cpu(), ref.leaky_forward(x.contiguous(), v0, a))


def test_empty_inputs_are_noops(hip):
    z = torch.zeros(0, device="cuda")
    assert hip.leakyForward(torch.zeros(0, 5, device="cuda"), z, z).shape == (0, 5)
    out = hip.leakyForward(torch.zeros(3, 0, device="cuda"), torch.zeros(3, device="cuda"), torch.ones(3, device="cuda"))
    assert out.shape == (3, 0)
    gi, ga, ginit = hip.leakyBackwardFused(torch.zeros(3, 0, device="cuda"), torch.ones(3, device="cuda"))
    assert gi.shape == (3, 0) and (ginit == 0).all()


def test_argument_errors(hip):
    x = torch.zeros(4, 8, device="cuda"); r = torch.zeros(4, device="cuda")
    with pytest.raises(RuntimeError):            # CPU tensor: there is no CPU path
        hip.leakyForward(torch.zeros(4, 8), torch.zeros(4), torch.zeros(4))
    with pytest.raises(RuntimeError):            # non-contiguous
        hip.leakyForward(torch.zeros(8, 4, device="cuda").t(), r, r)
    with pytest.raises(RuntimeError):            # wrong per-row length
        hip.leakyForward(x, torch.zeros(5, device="cuda"), r)
    with pytest.raises(RuntimeError):            # wrong dtype
        hip.leakyForward(x.double(), r.double(), r.double())
    with pytest.raises(RuntimeError):            # raw ABI: bad surrogate kind is rejected on the host
        hip.lifBackwardFused(x, None, x, None, r, r, r, None, False, -1, 17)


def test_one_way_streaming_probes():
    """bench.py's measurement probes (a library of their own, not part of libexodus_hip.so): the copy
    copies, the write probe zeroes exactly its range, the read probe writes nothing."""
    import bench
    probes = bench.Probes(torch)
    n = 4 * 1000 + 4
    buf = torch.full((n + 8,), 3.0, device="cuda")
    probes.write(buf[4:4 + n])
    assert bool((buf[4:4 + n] == 0).all()) and bool((buf[:4] == 3).all()) and bool((buf[4 + n:] == 3).all())
    a = torch.randn(n, device="cuda"); keep = a.clone()
    probes.read(a)
    assert torch.equal(a, keep)
    b = torch.randn(n, device="cuda"); dst = torch.empty(n, device="cuda")
    probes.stream(dst, a)
    assert torch.equal(dst, a)
    probes.stream(dst, a, b)
    assert torch.equal(dst, a + b)


@pytest.mark.parametrize("n,t", [(64, 1 << 22), (65, (1 << 22) - 4), (3, (1 << 22) + 4)])
def test_longest_rows_of_the_span_driver_and_the_first_beyond(hip, ref, n, t):
    """Rows of 2^22 steps: a wave's 64 rows are exactly the 2^30 bytes that the raw-buffer driver's 32-bit
    offsets cover; 2^22 - 4 steps puts row boundaries inside 64-byte sectors at that size; rows of 2^22 + 4 steps
    take the driver with full address arithmetic.  Leaky integrator forward and its reverse pass, bit for bit."""
    g = gen(t % 1000 + n)
    x = torch.randn(n, t, generator=g) * 0.3; v0 = torch.randn(n, generator=g)
    a = 0.9 + 0.1 * torch.rand(n, generator=g)
    out = hip.leakyForward(D(x), D(v0), D(a))
    want = ref.leaky_forward(x, v0, a)
    assert torch.equal(out.cpu(), want)
    del out
    gi = hip.leakyBackward(D(x), D(a))                       # the same tensor as incoming gradient
    assert torch.equal(gi.cpu(), ref.leaky_backward(x, a))
