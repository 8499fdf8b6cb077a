"""The two drivers of the (rows, time) kernels against each other with the whole GPU busy.

``test_gpu_rows_drivers.py`` compares them on at most 300 rows (5 waves).  The driver on raw buffer addressing carries
a guard behind its 16-byte stores (a short wait that keeps the data registers untouched until the store has read
them); the fault it guards against was only ever seen with several workgroups resident on a compute unit.  Here both
drivers run at 262 144 x 1000 (rows that start inside 64-byte sectors: the path that writes shared sectors in one piece)
and at 1 048 576 x 2000 (rows on sector boundaries; offsets beyond 2^31 elements) -- thousands of workgroups, every
compute unit full -- and every (rows, time) output is compared on the device, element for element: the same data once
16-byte aligned (raw buffer driver) and once one element further (the driver with full address arithmetic, itself
checked against the C oracle in test_gpu_kernels.py / test_gpu_rows_sweep.py / test_gpu_fullsize.py)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def placed(z, offset):
    """A copy of ``z`` that starts ``offset`` elements into a fresh allocation (allocations are 256-byte aligned)."""
    buf = torch.empty(z.numel() + 64, device=z.device)
    view = buf[offset:offset + z.numel()].view(z.shape)
    view.copy_(z)
    return view


def blank(shape, offset, dev):
    buf = torch.empty(shape[0] * shape[1] + 64, device=dev)
    return buf[offset:offset + shape[0] * shape[1]].view(shape)


@pytest.mark.parametrize("n,t", [(262144, 1000), (1 << 20, 2000)])
def test_span_driver_equals_generic_driver_with_every_compute_unit_full(n, t):
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip as hip
    free, _ = torch.cuda.mem_get_info()
    if free < 14 * n * t * 4:
        pytest.skip("not enough free device memory for both copies of every tensor")
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(n % 1000 + t)
    x = torch.randn(n, t, generator=g, device=dev) * 0.6 + 0.2
    go = torch.randn(n, t, generator=g, device=dev)
    am = 0.5 + 0.5 * torch.rand(n, generator=g, device=dev)
    a_s = 0.3 + 0.6 * torch.rand(n, generator=g, device=dev)
    th = 0.5 + torch.rand(n, generator=g, device=dev)
    c = th * (0.4 + 0.6 * torch.rand(n, generator=g, device=dev))
    lo = -0.2 - torch.rand(n, generator=g, device=dev)
    v0 = torch.randn(n, generator=g, device=dev) * 0.3
    i0 = torch.randn(n, generator=g, device=dev) * 0.3
    kind, p0, p1 = hip.SURR_SINGLE_EXP, 0.5, 1.0

    def both(run):
        """``run(offset)`` -> dict of outputs; with the aligned tensors (raw buffer driver) and one element further."""
        a, b = run(0), run(1)
        assert a.keys() == b.keys()
        for k in a:
            if k.endswith("~"):
                # per-row sums of t products, folded tile by tile in fp32 -- and the two drivers cut the tiles at different
                # steps.  Judged against a bound on the summed magnitudes, sum_t |adjoint_t| * max_t |state_t|: 16 fp32 ulps
                # of it, next to rtol 1e-4 (among a million rows some sums cancel to almost nothing)
                bound = a[k + " bound"]
                assert bool(((a[k] - b[k]).abs() <= 1e-4 * b[k].abs() + bound * 2.0 ** -20).all()), f"{k} at {n} x {t}"
            elif k.endswith(" bound"):
                continue
            else:
                if a[k].ndim == 2:
                    assert a[k].data_ptr() % 16 == 0 and b[k].data_ptr() % 16 == 4
                assert torch.equal(a[k], b[k]), f"{k} differs between the drivers at {n} x {t}"
        return a

    def spiking(o):
        xs = placed(x, o)
        s, v = blank((n, t), o, dev), blank((n, t), o, dev)
        hip.lifForward(s, v, xs, v0, am, c, th, lo, True, 2)
        gi = blank((n, t), o, dev)
        _, ga, g0 = hip.lifBackwardFused(placed(go, o), None, v, v0, am, c, th, lo, True, 2, kind, p0, p1,
                                         needAlphaGrad=True, inputGrad=gi)
        return {"lif spikes": s, "lif v_mem": v, "lif grad input": gi, "lif grad alpha~": ga, "lif grad init": g0,
                "lif grad alpha~ bound": gi.abs().sum(1) * (v.abs().amax(1) + 2 * c)}

    first = both(spiking)
    assert first["lif spikes"].sum().item() > n                # something to get wrong
    del first

    def leaky(o):
        xs = placed(x, o)
        out = blank((n, t), o, dev)
        hip.leakyForward(xs, v0, am, output=out)
        gi = blank((n, t), o, dev)
        _, ga, g0 = hip.leakyBackwardFused(placed(go, o), am, output=out, vmemInitial=v0, needAlphaGrad=True, inputGrad=gi)
        return {"leaky out": out, "leaky grad input": gi, "leaky grad alpha~": ga, "leaky grad init": g0,
                "leaky grad alpha~ bound": gi.abs().sum(1) * out.abs().amax(1)}

    both(leaky)

    def synaptic(o):
        xs = placed(x, o)
        s, v, i = (blank((n, t), o, dev) for _ in range(3))
        hip.synLifForward(xs, v0, i0, am, a_s, c, th, lo, True, 2, True, True, out=(s, v, i))
        gi = blank((n, t), o, dev)
        r = hip.synLifBackward(placed(go, o), None, None, v, i, v0, i0, am, a_s, c, th, lo, True, 2, True, True, kind, p0,
                               p1, inputGrad=gi)
        # (the adjoints behind these sums are grad_input up to the factors alpha_syn and 1 - alpha_mem, both below 1:
        # dividing by the smallest alpha_syn, 0.3, and by 0.5 x 0.3 bounds them)
        adjoint = gi.abs().sum(1) / 0.15
        return {"syn spikes": s, "syn v_mem": v, "syn i_syn": i, "syn grad input": gi, "syn grad alpha_mem~": r[1],
                "syn grad alpha_syn~": r[2], "syn grad v_init": r[3], "syn grad i_init": r[4],
                "syn grad alpha_mem~ bound": adjoint * (v.abs().amax(1) + 2 * c + i.abs().amax(1)),
                "syn grad alpha_syn~ bound": adjoint * (i.abs().amax(1) + xs.abs().amax(1))}

    both(synaptic)
