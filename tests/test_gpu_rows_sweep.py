"""Seeded sweep through the (rows, time) entry points against the C restatement of the reference kernels:
random row counts and lengths (around the 64-row waves and the 32-step tiles), matrices that start at element
offsets 0-3, 4 and 12 inside a larger buffer (16-byte vector accesses next to unaligned rows; rows that share
64-byte sectors, which the kernels then write in one piece), caps, clamp, the three
in-kernel surrogates, with and without a gradient on the membrane potential.  Forward outputs bit for bit;
gradients within rtol 1e-4 / atol 1e-5 (alpha gradients: atol scaled by sqrt(T)) plus 1e-5 of the largest magnitude."""
import random

import pytest
import torch

from _util import gen, note_scaled

pytestmark = pytest.mark.gpu


def excess(got, want, rtol=1e-4, atol=1e-5, of_max=1e-5):
    if not got.numel():
        return 0.0
    got = got.detach().cpu().double(); want = want.detach().double()
    return float(((got - want).abs() / (atol + rtol * want.abs() + of_max * want.abs().max())).max())


def test_random_rows_against_the_c_oracle():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip as hip
    from oracle import exodus_ref as ref
    rnd = random.Random(77)
    D = lambda z: None if z is None else z.cuda()
    worst = 0.0
    for case in range(300):
        n = rnd.choice([1, 2, 3, 63, 64, 65, 100, 127, 128, 129, 200, 256, 300, 513])
        t = rnd.choice([1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 36, 44, 47, 63, 64, 65, 68, 96, 100, 127, 128, 129, 132, 200,
                        260, 300, 301, 303])
        off = rnd.choice([0, 0, 0, 1, 2, 3, 4, 12])       # 4, 12: 16-byte aligned, but rows start inside 64-byte sectors
        g = gen(9000 + case)
        use_lo = rnd.random() < 0.6
        cap = rnd.choice([-1, 1, 2, 3])
        x = torch.randn(n, t, generator=g) * 0.7 + 0.25
        alpha = 0.5 + 0.5 * torch.rand(n, generator=g); v0 = torch.randn(n, generator=g) * 0.3
        th = 0.5 + torch.rand(n, generator=g); c = th * (0.4 + 0.6 * torch.rand(n, generator=g))
        lo = -0.2 - torch.rand(n, generator=g)
        what = f"case {case}: n={n} t={t} offset={off} clamp={use_lo} cap={cap}"

        def on_device(z):                                  # a device copy that starts `off` elements into a buffer
            buf = torch.empty(z.numel() + 16, device="cuda")
            view = buf[off:off + z.numel()].view(z.shape)
            view.copy_(z)
            return view

        want_s, want_v = ref.lif_forward(x, v0, alpha, c, th, lo if use_lo else None, use_lo, cap)
        xs = on_device(x); spikes = on_device(torch.zeros(n, t)); v_mem = on_device(torch.zeros(n, t))
        hip.lifForward(spikes, v_mem, xs, D(v0), D(alpha), D(c), D(th), D(lo) if use_lo else None, use_lo, cap)
        assert torch.equal(spikes.cpu(), want_s) and torch.equal(v_mem.cpu(), want_v), what
        go = torch.rand(n, t, generator=g)
        gv = torch.rand(n, t, generator=g) * 0.1 if rnd.random() < 0.5 else None
        kind, fn, p0 = rnd.choice([(hip.SURR_SINGLE_EXP, ref.SingleExponential(), 0.5),
                                   (hip.SURR_PERIODIC_EXP, ref.PeriodicExponential(), 0.5),
                                   (hip.SURR_HEAVISIDE, ref.Heaviside(0.6), 0.6)])
        want = ref.integrate_and_fire_backward(go, gv, want_v, want_s, v0, alpha, c, th, lo if use_lo else None, fn, True,
                                               gate_initial=True)
        got = hip.lifBackwardFused(on_device(go), None if gv is None else on_device(gv), v_mem, D(v0), D(alpha), D(c),
                                   D(th), D(lo) if use_lo else None, use_lo, cap, kind, p0, 1.0, needAlphaGrad=True)
        for name, a, b, atol in zip(("grad input", "grad alpha", "grad init"), got, want,
                                    (1e-5, 1e-5 * max(1, t) ** 0.5, 1e-5)):
            e = excess(a, b, atol=atol)
            note_scaled(f"rows sweep: {name}", a, b, 1e-4, atol, e)   # also in units of the plain rtol 1e-4 / atol 1e-5
            assert e <= 1, f"{what}: {name} {e:.3g} x tolerance"
            worst = max(worst, e)
        want_o = ref.leaky_forward(x, v0, alpha)
        out = hip.leakyForward(xs, D(v0), D(alpha))
        assert torch.equal(out.cpu(), want_o), what
        want = ref.leaky_integrator_backward(go, want_o, v0, alpha, True)
        got = hip.leakyBackwardFused(on_device(go), D(alpha), out, D(v0), True)
        for name, a, b, atol in zip(("leaky grad input", "leaky grad alpha", "leaky grad init"), got, want,
                                    (1e-5, 1e-5 * max(1, t) ** 0.5, 1e-5)):
            e = excess(a, b, atol=atol)
            note_scaled(f"rows sweep: {name}", a, b, 1e-4, atol, e)   # also in units of the plain rtol 1e-4 / atol 1e-5
            assert e <= 1, f"{what}: {name} {e:.3g} x tolerance"
            worst = max(worst, e)
    print(f"largest gradient difference: {worst:.3g} x tolerance")
