"""Region-aware allocation (sinabs.exodus.hbm): three ranges are made of one region of HBM each (checked by
timed copies), a fourth alternates between the regions page by page (checked by what a kernel gains from writing
into it), the layer wrappers put what they write into the striped range -- or, without one, into another region than
what they read -- and no result changes with where the tensors lie.  The reference has no
counterpart; its extension allocates outputs with ``torch.empty_like`` (reference cuda/bindings.cu:98,144,183)."""
import os

import pytest
import torch

from _util import gen

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture()
def hbm():
    assert torch.cuda.is_available()
    from sinabs.exodus import hbm as module
    torch.cuda.empty_cache()
    yield module
    module.disable()
    torch.cuda.empty_cache()


def sorted_ranges(hbm, **sizes):
    """The ranges -- or a skip when this machine's free memory no longer shows regions: a process that allocated and
    freed device memory in 64 MiB pages (the striped range is made of such) leaves it to later processes as a mixture
    of the regions below the 4 GiB the sorting judges, and then there is nothing to sort (a machine that has run
    nothing else, as at the start of a test run, is not in that state)."""
    try:
        regions = hbm.enable(**sizes)
    except RuntimeError as err:
        if "did not show three kinds" in str(err):
            pytest.skip("device memory comes back mixed from earlier processes: no regions to sort by")
        raise
    if not regions.verified:
        hbm.disable()
        pytest.skip(f"device memory comes back partly mixed from earlier processes: {regions.report}")
    return regions


def test_outputs_go_to_another_pool_and_results_do_not_change(hbm):
    """Ranges of single regions only (no striped range): the wrappers put what they write into another region than
    what they read.  Runs first: it allocates in chunks of 4 GiB only, which leaves the driver's memory in order."""
    from sinabs.exodus import _hip as hip
    dev = torch.device("cuda:0")
    B, T, M = 4, 300, 65536                                   # 300 MiB per tensor: large enough to be classified
    n = B * M
    x_plain = (torch.randn(B, T, M, generator=gen(3)) * 0.5 + 0.05).to(dev)
    go_plain = torch.rand(B, T, M, generator=gen(4)).to(dev)
    full = lambda v: torch.full((n,), float(v), device=dev)
    zeros = torch.zeros(n, device=dev)
    a_mem, a_syn, one, lo = full(0.95), full(0.8), full(1.0), full(-1.0)

    def run(x, go):
        f = hip.layerLifForward(x, zeros, zeros, a_mem, a_syn, one, one, lo, True, 2, True, True)
        g = hip.layerLifBackward(go, None, None, x, f["ckpt_v"], f["ckpt_i"], zeros, zeros, a_mem, a_syn, one, one,
                                 lo, True, 2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
        leak, _ = hip.layerLeakyForward(x, zeros, a_mem, False, False)
        gl = hip.layerLeakyBackward(go, None, leak, x, zeros, a_mem, False, False, True)
        return f, g, leak, gl

    want_f, want_g, want_leak, want_gl = run(x_plain, go_plain)
    assert want_f["spikes"].sum().item() > 0

    regions = sorted_ranges(hbm, gib_per_region=16.0, gib_striped=0.0)     # 4 chunks each: the check of the finished ranges averages over more copies
    assert hbm.active() is regions
    x = regions.empty((B, T, M), region=0).copy_(x_plain)
    go = regions.empty((B, T, M), region=0).copy_(go_plain)
    assert regions.pool_of(x) == 0 and regions.region_of(go) == 0 and regions.pool_of(x_plain) is None
    f, g, leak, gl = run(x, go)
    assert regions.pool_of(f["spikes"]) in (1, 2)
    assert regions.pool_of(f["ckpt_v"]) in (1, 2) and regions.pool_of(f["ckpt_v"]) != regions.pool_of(f["spikes"])
    assert regions.pool_of(g[0]) in (1, 2)                     # grad_input: away from grad_output and the input
    assert regions.pool_of(leak) in (1, 2)
    assert regions.pool_of(gl[0]) == 3 - regions.pool_of(leak)  # reads pool 0 and the output's pool, writes the third
    for k in ("spikes", "v_last", "i_last", "ckpt_v", "ckpt_i", "spike_sum"):
        assert torch.equal(f[k], want_f[k]), k
    for got, want in zip(list(g) + [leak] + list(gl), list(want_g) + [want_leak] + list(want_gl)):
        assert (got is None) == (want is None)
        if got is not None:
            assert torch.equal(got, want)

    # inputs from the ordinary allocator are classified by timed copies, once per storage; the result still
    # lands in one of the pools, and the values are the same
    k = regions.region_of(x_plain)
    assert k in (0, 1, 2) and regions.region_of(x_plain) == k
    f2 = hip.layerLifForward(x_plain, zeros, zeros, a_mem, a_syn, one, one, lo, True, 2, True, True)
    assert regions.pool_of(f2["spikes"]) not in (None, k)
    assert torch.equal(f2["spikes"], want_f["spikes"])
    small = torch.zeros(2, 8, 64, device=dev)
    assert regions.region_of(small) is None                    # too small to time or to matter

    hbm.disable()
    assert hbm.active() is None
    again = hip.layerLifForward(x_plain, zeros, zeros, a_mem, a_syn, one, one, lo, True, 2, True, True)
    assert torch.equal(again["spikes"], want_f["spikes"])


def test_ranges_of_one_region_each_and_a_striped_range_that_takes_writes_faster(hbm):
    """Copies between the regions' ranges beat copies inside one range, whatever this process and earlier ones have
    done to the order in which the driver hands out memory.  The striped range: the wrappers' outputs go there,
    results do not change, and a kernel that writes single 128-byte lines (the (rows, time) leaky integrator, one
    tensor in, one out) is clearly faster into it than into one region (measured 5.6-5.7 against 4.6-4.9 TB/s)."""
    from sinabs.exodus import _hip as hip
    dev = torch.device("cuda:0")
    regions = sorted_ranges(hbm, gib_per_region=16.0, gib_striped=24.0)
    rep = regions.report
    print(f"\n{rep}")
    inside, across = rep["inside_one_range_GBs"], rep["across_ranges_GBs"]
    assert rep["kinds_found"] == 3 and regions.verified is True
    assert sum(across) / 6 > 1.025 * sum(inside) / 3            # what `verified` says
    assert regions.sizes[hbm.STRIPED] == 24 * 2 ** 30 and regions.page_bytes == 64 * 2 ** 20
    spans = sorted(zip(regions.bases, regions.sizes))
    assert all(n == 16 * 2 ** 30 for _, n in spans if n != 24 * 2 ** 30)
    assert all(spans[k][0] + spans[k][1] <= spans[k + 1][0] for k in range(3))
    # tensors are views of the ranges, given back when released
    free = regions.bytes_free(1)
    t = regions.empty((3, 1000, 1000), region=1)
    assert regions.pool_of(t) == 1 and t.data_ptr() % (2 * 2 ** 20) == 0 and t.is_contiguous()
    assert regions.bytes_free(1) == free - 12 * 2 ** 20        # 12e6 bytes rounded up to 2 MiB pieces
    u = regions.empty((2 ** 20,), torch.float64, region=1)
    assert u.dtype == torch.float64 and regions.pool_of(u) == 1 and u.data_ptr() >= t.data_ptr() + 12 * 2 ** 20
    t.fill_(3.0); u.fill_(5.0)
    assert t.sum().item() == 9e6 and u.sum().item() == 5 * 2 ** 20
    del t, u
    assert regions.bytes_free(1) == free
    full = regions.empty((17 * 2 ** 30,), torch.uint8, region=2)   # more than the range holds: ordinary allocator
    assert regions.pool_of(full) is None
    del full

    n, t = 1048576, 1024                                       # 4 GiB per tensor
    x = regions.empty((n, t), region=0).normal_(0.0, 1.0, generator=torch.Generator(device=dev).manual_seed(5))
    alpha = torch.full((n,), 0.9, device=dev)
    zeros = torch.zeros(n, device=dev)
    one_region = regions.empty((n, t), region=1)
    striped = regions.empty((n, t))
    assert regions.pool_of(one_region) == 1 and regions.pool_of(striped) == hbm.STRIPED
    assert regions.region_of(striped) is None

    def rate(out):
        for _ in range(2):
            hip.leakyForward(x, zeros, alpha, output=out)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(7)]
        for a, b in ev:
            a.record()
            hip.leakyForward(x, zeros, alpha, output=out)
            b.record()
        torch.cuda.synchronize()
        return 8 * n * t / sorted(a.elapsed_time(b) for a, b in ev)[3] / 1e9

    into_one, into_striped = rate(one_region), rate(striped)
    print(f"leaky forward into one region {into_one:.2f} TB/s, into the striped range {into_striped:.2f} TB/s")
    assert torch.equal(one_region, striped)
    assert into_striped > 1.08 * into_one
    own = hip.leakyForward(x, zeros, alpha)                    # the wrapper's own allocation goes there as well
    assert regions.pool_of(own) == hbm.STRIPED and torch.equal(own, striped)
    del one_region, striped, own
    # the layer wrappers allocate in the striped range, and the values are what the ordinary allocator gives
    xs = x[:65536 * 4].view(4, 1024, 65536)
    f = hip.layerLifForward(xs, zeros[:4 * 65536], None, alpha[:4 * 65536], None, alpha[:4 * 65536] + 0.1,
                            alpha[:4 * 65536] + 0.1, None, False, 1, False, False)
    assert regions.pool_of(f["spikes"]) == hbm.STRIPED and regions.pool_of(f["ckpt_v"]) == hbm.STRIPED
    hbm.disable()
    plain = hip.layerLifForward(xs, zeros[:4 * 65536], None, alpha[:4 * 65536], None, alpha[:4 * 65536] + 0.1,
                                alpha[:4 * 65536] + 0.1, None, False, 1, False, False)
    assert hbm.active() is None and regions.pool_of(plain["spikes"]) is None
    assert torch.equal(plain["spikes"], f["spikes"]) and torch.equal(plain["ckpt_v"], f["ckpt_v"])
    assert f["spikes"].sum().item() > 0
    # closed with live tensors (x, f): the memory stays until the last one goes, new requests go elsewhere
    assert x[:4].sum().isfinite() and regions.pool_of(regions.empty((2 ** 20,), region=0)) is None


def test_striped_range_alone_is_made_of_whatever_memory_there_is(hbm):
    """Only a striped range: made whether or not the memory shows regions, usable, and given back."""
    regions = hbm.enable(gib_per_region=0.0, gib_striped=12.0)
    print(f"\nsorted: {regions.sorted}; {regions.report}")
    assert regions.sizes[:3] == [0, 0, 0] and regions.sizes[hbm.STRIPED] == 12 * 2 ** 30
    assert regions.verified == (regions.sorted and regions.verified)
    t = regions.empty((2 ** 30,))                             # 4 GiB across 64 pages
    assert regions.pool_of(t) == hbm.STRIPED and regions.region_of(t) is None
    t.copy_(torch.arange(2 ** 30, device=t.device, dtype=torch.int32) % 1024)
    assert t.view(-1, 1024).eq(torch.arange(1024, device=t.device, dtype=torch.float32)).all()
    u = regions.empty((3 * 2 ** 30,), region=1)               # no such range: the ordinary allocator
    assert regions.pool_of(u) is None
    del t, u
    hbm.disable()


def test_layers_and_functions_give_the_same_results_from_the_striped_range(hbm):
    """A small network of the public layers and the IntegrateAndFire Function, forward and backward, with and without
    ``hbm.enable()``: every output and gradient bit for bit the same (the range only changes where tensors lie)."""
    import torch.nn as nn
    import sinabs.exodus.layers as el
    from sinabs.exodus.spike import IntegrateAndFire
    from sinabs.exodus._compat import activation as act
    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    net = nn.Sequential(el.LIF(tau_mem=20.0, tau_syn=5.0, min_v_mem=-1.0, spike_fn=act.MaxSpike(2), train_alphas=True),
                        el.IAF()).to(dev)
    x = (torch.rand(8, 200, 4096, generator=gen(12)) * 0.8).to(dev).requires_grad_(True)    # 26 MB per tensor
    rows = (torch.randn(4096, 512, generator=gen(13)) * 0.6 + 0.2).to(dev)  # (rows, time) tensors of 8 MiB
    alpha = torch.full((4096,), 0.9, device=dev); ones = torch.ones(4096, device=dev)

    def run():
        for m in net:
            if hasattr(m, "reset_states"):
                m.reset_states()
        net.zero_grad(set_to_none=True)
        x.grad = None
        out = net(x)
        out.sum().backward()
        inp = rows.clone().requires_grad_(True)
        s, v = IntegrateAndFire.apply(inp, alpha, torch.zeros_like(alpha), ones, ones, None, act.SingleExponential(), None)
        (s.sum() + 0.1 * v.sum()).backward()
        return [out.detach(), x.grad, s.detach(), v.detach(), inp.grad] + [p.grad for p in net.parameters()], (out, s)

    want, _ = run()
    assert want[0].sum().item() > 0 and want[2].sum().item() > 0 and want[1].abs().sum().item() > 0
    regions = hbm.enable(gib_per_region=0.0, gib_striped=6.0, sort=False)
    got, (out, s) = run()
    assert regions.pool_of(s) == hbm.STRIPED and regions.pool_of(out) == hbm.STRIPED
    assert regions.pool_of(net[1].v_mem) is None               # states are small: the ordinary allocator
    same = lambda p, q: all((a is None and b is None) or torch.equal(a, b) for a, b in zip(p, q))
    assert len(got) == len(want) and same(got, want) and sum(g is not None for g in got) >= 7
    hbm.disable()
    again, _ = run()
    assert same(again, want)


def test_striped_range_without_sorting(hbm):
    """``sort=False``: no timed copies; the striped range is made of chunks spread evenly over the free memory --
    the same code that runs when the copies show no regions (memory left mixed by earlier processes) -- and holds
    what is written to it; ranges of single regions cannot be had that way."""
    regions = hbm.HbmRegions(gib_per_region=0.0, gib_striped=6.0, sort=False)
    print(f"\nsorted: {regions.sorted}; {regions.report}")
    assert regions.sorted is False and regions.verified is False and regions.report["kinds_found"] == 0
    assert regions.sizes[hbm.STRIPED] == 12 * 2 ** 30 and regions.sizes[:3] == [0, 0, 0]   # three chunks of 4 GiB
    t = regions.empty((2 ** 31,))                              # 8 GiB: pages of all three chunks
    assert regions.pool_of(t) == hbm.STRIPED
    pattern = torch.arange(2 ** 31, device=t.device, dtype=torch.int32) % 4099
    t.copy_(pattern)
    assert t.view(-1, 2 ** 15)[::37].eq(pattern.view(-1, 2 ** 15)[::37]).all()
    del t, pattern
    regions.close()
    with pytest.raises(ValueError):
        hbm.HbmRegions(gib_per_region=1.0, gib_striped=0.0, sort=False)


def test_too_little_free_memory_is_refused(hbm):
    with pytest.raises(ValueError):
        hbm.HbmRegions(gib_per_region=96.0)
    free, _ = torch.cuda.mem_get_info()
    held = torch.empty(free - 40 * 2 ** 30, dtype=torch.uint8, device="cuda:0")
    with pytest.raises(RuntimeError, match="out of memory"):
        hbm.HbmRegions(gib_per_region=8.0, gib_striped=0.0)
    del held
    assert hbm.active() is None
