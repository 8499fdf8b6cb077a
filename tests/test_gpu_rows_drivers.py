"""The two drivers of the (rows, time) kernels against each other, through every entry point: the same data once in
16-byte aligned tensors (element offsets 0, 4, 8, ... inside a larger buffer: the driver on raw buffer addressing,
which also writes the 64-byte sectors shared by two rows in one piece) and once one element further (the driver with
full address arithmetic).  Same arithmetic in the same order: all (rows, time) outputs bit for bit, per-row sums
(folded per tile, and the tiles differ) within tolerance; buffers are filled with NaN around the tensors, and nothing
outside a tensor may be written.  The second driver is itself checked against the C oracle
(test_gpu_kernels.py, test_gpu_rows_sweep.py)."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_span_driver_equals_generic_driver_on_every_entry_point():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip as hip
    dev = "cuda"
    rnd = random.Random(5)

    def at(z, off):
        buf = torch.full((z.numel() + 64,), float("nan"), device=dev)
        view = buf[off:off + z.numel()].view(z.shape)
        view.copy_(z)
        return view, buf

    def untouched(buf, off, numel):
        return bool(torch.isnan(buf[:off]).all() and torch.isnan(buf[off + numel:]).all())

    for case in range(250):
        n = rnd.choice([1, 2, 63, 64, 65, 100, 127, 128, 129, 192, 200, 257, 300])
        t = 4 * rnd.choice([1, 2, 3, 4, 7, 8, 9, 10, 11, 12, 13, 15, 16, 17, 19, 24, 25, 31, 32, 33, 50, 75, 77, 100, 125])
        off = 4 * rnd.choice([0, 0, 1, 2, 3, 4, 5, 7])
        g = torch.Generator().manual_seed(9176 + case)
        use_lo = rnd.random() < 0.6
        cap = rnd.choice([-1, 1, 2, 3])
        de, ni = rnd.random() < 0.5, rnd.random() < 0.5
        R = lambda *s, sc=1.0, o=0.0: (torch.randn(*s, generator=g) * sc + o).to(dev)
        x = R(n, t, sc=0.7, o=0.25); go = R(n, t); gv = R(n, t, sc=0.1); gq = R(n, t, sc=0.1)
        am = (0.5 + 0.5 * torch.rand(n, generator=g)).to(dev); a_s = (0.3 + 0.6 * torch.rand(n, generator=g)).to(dev)
        v0 = R(n, sc=0.3); i0 = R(n, sc=0.3); th = (0.5 + torch.rand(n, generator=g)).to(dev)
        c = th * (0.4 + 0.6 * torch.rand(n, generator=g)).to(dev); lo = (-0.2 - torch.rand(n, generator=g)).to(dev)
        low = lo if use_lo else None
        what = f"case {case}: n={n} t={t} offset={off} clamp={use_lo} cap={cap} decay_early={de} norm_input={ni}"
        res = {}
        for tag, o in (("span", off), ("generic", off + 1)):
            r = {}
            xs, _ = at(x, o); gos, _ = at(go, o); gvs, _ = at(gv, o); gqs, _ = at(gq, o)
            sp, bsp = at(torch.zeros(n, t), o); vm, bvm = at(torch.zeros(n, t), o)
            hip.lifForward(sp, vm, xs, v0, am, c, th, low, use_lo, cap)
            r["lif spikes"], r["lif v_mem"] = sp.clone(), vm.clone()
            ok = untouched(bsp, o, n * t) and untouched(bvm, o, n * t)
            gi, bgi = at(torch.zeros(n, t), o)
            _, ga, g0 = hip.lifBackwardFused(gos, gvs if case % 2 else None, vm, v0, am, c, th, low, use_lo, cap,
                                             hip.SURR_SINGLE_EXP, 0.5, 1.0, needAlphaGrad=True, inputGrad=gi)
            r["lif grad input"], r["lif grad alpha~"], r["lif grad init"] = gi.clone(), ga, g0
            ok = ok and untouched(bgi, o, n * t)
            out, bout = at(torch.zeros(n, t), o)
            hip.leakyForward(xs, v0, am, output=out)
            r["leaky out"] = out.clone()
            gil, bgil = at(torch.zeros(n, t), o)
            _, gal, g0l = hip.leakyBackwardFused(gos, am, output=out, vmemInitial=v0, needAlphaGrad=True, inputGrad=gil)
            r["leaky grad input"], r["leaky grad alpha~"], r["leaky grad init"] = gil.clone(), gal, g0l
            ok = ok and untouched(bout, o, n * t) and untouched(bgil, o, n * t)
            three = [at(torch.zeros(n, t), o) for _ in range(3)]
            hip.synLifForward(xs, v0, i0, am, a_s, c, th, low, use_lo, cap, de, ni, out=tuple(a for a, _ in three))
            r["syn spikes"], r["syn v_mem"], r["syn i_syn"] = (a.clone() for a, _ in three)
            ok = ok and all(untouched(b, o, n * t) for _, b in three)
            gis, bgis = at(torch.zeros(n, t), o)
            extra = case % 3 == 0
            rr = hip.synLifBackward(gos, gvs if extra else None, gqs if extra else None, three[1][0], three[2][0], v0, i0,
                                    am, a_s, c, th, low, use_lo, cap, de, ni, hip.SURR_SINGLE_EXP, 0.5, 1.0, inputGrad=gis)
            r["syn grad input"] = gis.clone()
            r["syn grad alpha_mem~"], r["syn grad alpha_syn~"], r["syn grad v_init"], r["syn grad i_init"] = rr[1:]
            ok = ok and untouched(bgis, o, n * t)
            pv, bpv = at(x * 2.0, o)
            r["spike function spikes"] = hip.spikeForward(pv, 0.9, 0.8, 1.0, -0.5, use_lo, cap)    # v_mem in place
            r["spike function v_mem"] = pv.clone()
            ok = ok and untouched(bpv, o, n * t)
            mask = (xs > -0.3).float()
            r["spike function grad"] = hip.spikeBackward(gvs.abs(), gos, mask, 0.9, 0.8)
            r["lifBackward"] = hip.lifBackward(gvs.abs(), gos, mask, am, am * c)
            r["lifBackwardAlpha~"] = hip.lifBackwardAlpha(gvs.abs(), gos, vm, v0, mask, am, c)
            r["nothing written outside the tensors"] = ok
            res[tag] = r
        for k, a in res["span"].items():
            b = res["generic"][k]
            if isinstance(a, bool):
                assert a and b, f"{what}: {k}"
            elif k.endswith("~"):
                assert torch.allclose(a, b, rtol=1e-4, atol=1e-5 * max(1, t) ** 0.5), f"{what}: {k}"
            else:
                assert torch.equal(a, b), f"{what}: {k}"
