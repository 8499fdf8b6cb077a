"""Region-aware allocation (sinabs.exodus.hbm): a range of device memory whose 64 MiB pages alternate between the
regions of HBM backs a ``torch.cuda.MemPool``; the layer wrappers put what they write there, ``placement()`` and
``enable(everything=True)`` send torch's own allocations there too, and no result changes with where the tensors
lie.  The reference has no counterpart; its extension allocates outputs with ``torch.empty_like`` (reference
cuda/bindings.cu:98,144,183).

Nothing here asserts on a measured rate: what the placement is worth is reported by ``bench.py``
(``roofline.frac_by_placement``, ``others[*].ordinary_allocator``)."""
import ctypes
import gc
import os

import pytest
import torch

from _util import gen

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MIB, GIB = 2 ** 20, 2 ** 30


@pytest.fixture()
def hbm():
    assert torch.cuda.is_available()
    from sinabs.exodus import hbm as module
    gc.collect()
    torch.cuda.empty_cache()
    assert module.disable(), "an earlier test left tensors alive in its ranges"
    yield module
    gc.collect()
    assert module.disable(), "this test left tensors alive in its ranges"
    torch.cuda.empty_cache()


def network_and_data(dev):
    import torch.nn as nn
    import sinabs.exodus.layers as el
    from sinabs.exodus._compat import activation as act
    torch.manual_seed(3)
    net = nn.Sequential(el.LIF(tau_mem=20.0, tau_syn=5.0, min_v_mem=-1.0, spike_fn=act.MaxSpike(2), train_alphas=True),
                        el.IAF()).to(dev)
    x = (torch.rand(8, 200, 4096, generator=gen(12)) * 0.8).to(dev).requires_grad_(True)    # 26 MB per tensor
    rows = (torch.randn(4096, 512, generator=gen(13)) * 0.6 + 0.2).to(dev)  # (rows, time) tensors of 8 MiB
    return net, x, rows


def run_network(net, x, rows, weights=None):
    """Forward and backward through two layers and the IntegrateAndFire Function; returns every output and gradient
    (and the live output tensors, for looking at where they lie)."""
    from sinabs.exodus.spike import IntegrateAndFire
    from sinabs.exodus._compat import activation as act
    dev = x.device
    alpha = torch.full((4096,), 0.9, device=dev); ones = torch.ones(4096, device=dev)
    for m in net:
        if hasattr(m, "reset_states"):
            m.reset_states()
    net.zero_grad(set_to_none=True)
    x.grad = None
    seen = {}
    mid = net[0](x)
    mid.register_hook(lambda g: seen.__setitem__("grad_mid", g))
    out = net[1](mid * 1.5)
    out.register_hook(lambda g: seen.__setitem__("grad_out", g))
    loss = out.sum() if weights is None else (out * weights).sum()
    loss.backward()
    inp = rows.clone().requires_grad_(True)
    s, v = IntegrateAndFire.apply(inp, alpha, torch.zeros_like(alpha), ones, ones, None, act.SingleExponential(), None)
    (s.sum() + 0.1 * v.sum()).backward()
    values = [out.detach(), x.grad, s.detach(), v.detach(), inp.grad] + [p.grad for p in net.parameters()]
    return values, dict(out=out, mid=mid, s=s, **seen)


def same(p, q):
    return len(p) == len(q) and all((a is None and b is None) or torch.equal(a, b) for a, b in zip(p, q))


def test_wrappers_allocate_in_the_striped_range_and_results_do_not_change(hbm):
    """A small network of the public layers and the IntegrateAndFire Function, forward and backward, with and without
    ``hbm.enable()``: every output and gradient bit for bit the same (the range only changes where tensors lie),
    big outputs in the striped range, small ones and the program's own tensors where they were."""
    dev = torch.device("cuda:0")
    net, x, rows = network_and_data(dev)
    want = run_network(net, x, rows)[0]
    assert want[0].sum().item() > 0 and want[2].sum().item() > 0 and want[1].abs().sum().item() > 0
    regions = hbm.enable(gib_striped=6.0)
    print(f"\nset-up {regions.setup_s:.2f} s; {regions.report}")
    assert hbm.active() is regions and regions.sorted is False and regions.report["kinds_found"] == 0
    assert regions.sizes[:3] == [0, 0, 0] and regions.sizes[hbm.STRIPED] == 12 * GIB and regions.page_bytes == 64 * MIB
    got, live = run_network(net, x, rows)
    assert regions.pool_of(live["s"]) == hbm.STRIPED and regions.pool_of(live["out"]) == hbm.STRIPED
    assert regions.pool_of(live["mid"]) == hbm.STRIPED
    assert regions.pool_of(x.grad) == hbm.STRIPED              # grad_input of the first layer: written by the kernel
    assert regions.pool_of(x) is None and regions.pool_of(rows) is None   # the program's own tensors
    assert regions.pool_of(net[1].v_mem) is None               # states are small: the ordinary allocator
    assert same(got, want) and sum(g is not None for g in got) >= 7
    assert regions.bytes_in_use() > 0 and regions.bytes_elsewhere() == 0
    del got, live
    # tensors alive in the ranges: they cannot be given back yet, and new ranges cannot be made
    keep = hbm.empty((4, MIB), x)
    assert regions.pool_of(keep) == hbm.STRIPED
    assert hbm.disable() is False and hbm.active() is None
    keep.fill_(2.0)
    assert keep.sum().item() == 8.0 * MIB                      # still mapped, still usable
    with pytest.raises(RuntimeError, match="still alive"):
        hbm.enable(gib_striped=6.0)
    again, live = run_network(net, x, rows)                    # not enabled any more: the ordinary allocator
    assert same(again, want) and regions.pool_of(live["out"]) is None
    del keep, again, live, net, x
    gc.collect()
    assert hbm.disable() is True


def test_the_pool_behaves_like_any_memory_of_the_caching_allocator(hbm):
    """Blocks are reused, split and kept apart by stream as PyTorch's allocator does with ordinary memory; a range
    that is full hands out ordinary memory instead of failing."""
    dev = torch.device("cuda:0")
    like = torch.empty(1, device=dev)
    regions = hbm.enable(gib_striped=6.0)                      # three chunks of 4 GiB
    a = hbm.empty((256, 1024, 1024), like)                     # 1 GiB
    assert regions.pool_of(a) == hbm.STRIPED and a.data_ptr() % (2 * MIB) == 0 and a.is_contiguous()
    assert regions.bytes_in_use() == GIB
    small = hbm.empty((16,), like)
    assert regions.pool_of(small) is None                      # below 1 MiB: not worth placing
    p = a.data_ptr()
    del a
    assert regions.bytes_in_use() == GIB                       # cached by PyTorch, not returned
    b = hbm.empty((256, 1024, 1024), like)
    assert b.data_ptr() == p                                   # ... and handed out again
    u = regions.empty((MIB,), torch.float64)
    assert u.dtype == torch.float64 and regions.pool_of(u) == hbm.STRIPED
    b.fill_(3.0); u.fill_(5.0)
    assert b.sum().item() == 3.0 * 2 ** 28 and u.sum().item() == 5.0 * MIB
    # a block that another stream still uses is not handed out again before that stream is done with it
    side = torch.cuda.Stream()
    big = hbm.empty((512, 1024, 1024), like).fill_(1.0)        # 2 GiB
    pb = big.data_ptr()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(60):
            big.mul_(1.0001)
    big.record_stream(side)
    del big
    nxt = hbm.empty((512, 1024, 1024), like)                   # while the side stream is still multiplying
    assert nxt.data_ptr() != pb and regions.pool_of(nxt) == hbm.STRIPED
    side.synchronize()
    del nxt, b, u
    # no such range: the ordinary allocator
    v = regions.empty((3 * MIB,), region=1)
    assert regions.pool_of(v) is None
    with pytest.raises(ValueError):
        regions.pool(1)
    # a request beyond what the range holds is served from ordinary memory, which the pool keeps like its own
    whole = regions.empty((13 * GIB,), torch.uint8)
    assert regions.pool_of(whole) is None and regions.bytes_elsewhere() >= 13 * GIB
    whole[:: GIB].fill_(7)
    assert int(whole[:: GIB].sum().item()) == 7 * 13
    del whole, v, small, like
    gc.collect()
    assert hbm.disable() is True                               # the pool goes, and with it what it had cached
    assert regions.bytes_elsewhere() == 0 and regions.bytes_in_use() == 0


def test_placement_block_and_everything_mode_cover_what_torch_allocates(hbm):
    """``with hbm.placement():`` -- this thread's allocations come from the striped range, nested wrapper calls
    included.  ``enable(everything=True)`` -- every thread's, among them the gradient tensors that autograd's own
    thread allocates during a backward pass; values stay bit-identical."""
    dev = torch.device("cuda:0")
    net, x, rows = network_and_data(dev)
    weights = torch.rand(8, 200, 4096, generator=gen(14)).to(dev)
    want = run_network(net, x, rows, weights)[0]        # (only the values: the live tensors' graphs hold x and the parameters)
    regions = hbm.enable(gib_striped=6.0)
    with hbm.placement():
        t = torch.randn(64, 1024, 1024, device=dev)
        u = t * 2
        inner = hbm.empty_like(t)                              # a wrapper's request inside the block
    outside = torch.randn(64, 1024, 1024, device=dev)
    assert [regions.pool_of(v) for v in (t, u, inner, outside)] == [hbm.STRIPED] * 3 + [None]
    got, live = run_network(net, x, rows, weights)
    # the gradient of the last layer's output is made by torch (the backward of the product with `weights`), in
    # autograd's thread: not covered by wrappers or by a placement block of the main thread
    assert regions.pool_of(live["grad_out"]) is None and regions.pool_of(live["grad_mid"]) is None
    assert same(got, want)
    del t, u, inner, outside, got, live
    x.grad = None                                              # written by the first layer's kernel: lies in the range
    gc.collect()
    assert hbm.disable() is True

    regions = hbm.enable(gib_striped=6.0, everything=True)
    y = torch.randn(4, 1024, 1024, device=dev)
    assert regions.pool_of(y) == hbm.STRIPED
    got, live = run_network(net, x, rows, weights)
    assert regions.pool_of(live["grad_out"]) == hbm.STRIPED    # torch-made, autograd's thread
    assert regions.pool_of(live["grad_mid"]) == hbm.STRIPED    # torch-made: the backward of `mid * 1.5`
    assert regions.pool_of(live["out"]) == hbm.STRIPED and regions.pool_of(x.grad) == hbm.STRIPED
    assert same(got, want)
    del y, got, live, net, x, rows, weights, want
    gc.collect()
    assert hbm.disable() is True, regions.live_blocks()
    z = torch.randn(4, 1024, 1024, device=dev)
    assert regions.pool_of(z) is None


def test_pieces_of_the_ranges_through_the_c_abi(hbm):
    """exodus_hbm_alloc_striped / exodus_hbm_free as a caller without PyTorch would use them: first fit from the
    lowest address in pieces of 2 MiB, neighbours joined on release, ordinary memory when the range is full or absent,
    and ranges that still have pieces out are not destroyed."""
    from sinabs.exodus import _hip
    lib = _hip.lib
    dev = torch.device("cuda:0")
    used = (ctypes.c_uint64 * 4)()
    other = ctypes.c_uint64(0)
    usage = lambda: (lib.exodus_hbm_usage(0, used, ctypes.byref(other)), list(used), other.value)[1:]
    # no ranges: plain device memory, given back by the same free
    p = lib.exodus_hbm_alloc_striped(3 * MIB, 0, None)
    assert p and usage() == ([0, 0, 0, 0], 3 * MIB)
    lib.exodus_hbm_free(p, 3 * MIB, 0, None)
    assert usage() == ([0, 0, 0, 0], 0)
    lib.exodus_hbm_free(ctypes.c_void_p(4096), 1, 0, None)     # not handed out by the library: ignored
    regions = hbm.HbmRegions(gib_striped=6.0)
    base, size = regions.bases[hbm.STRIPED], regions.sizes[hbm.STRIPED]
    a = lib.exodus_hbm_alloc_striped(3 * MIB, 0, None)         # rounded up to 4 MiB
    b = lib.exodus_hbm_alloc_striped(2 * MIB, 0, None)
    c = lib.exodus_hbm_alloc_striped(size - 6 * MIB, 0, None)
    assert (a, b, c) == (base, base + 4 * MIB, base + 6 * MIB) and usage() == ([0, 0, 0, size], 0)
    d = lib.exodus_hbm_alloc_striped(1, 0, None)               # full: ordinary memory
    assert d and not base <= d < base + size and usage()[1] == 1
    assert lib.exodus_hbm_regions_destroy(0) == hbm.RANGE_IN_USE
    assert "has not come back" in lib.exodus_hip_error_string(hbm.RANGE_IN_USE).decode()
    t = torch.as_tensor(_Bytes(a, 4 * MIB), device=dev)        # the memory is real
    t.fill_(9)
    assert int(t.sum().item()) == 9 * 4 * MIB
    del t
    torch.cuda.synchronize()
    lib.exodus_hbm_free(b, 2 * MIB, 0, None)
    lib.exodus_hbm_free(a, 3 * MIB, 0, None)                   # joins the piece behind it
    assert lib.exodus_hbm_alloc_striped(5 * MIB, 0, None) == base
    lib.exodus_hbm_free(c, size - 6 * MIB, 0, None)
    lib.exodus_hbm_free(base, 5 * MIB, 0, None)                # joins the piece after it: one free range again
    lib.exodus_hbm_free(d, 1, 0, None)
    assert usage() == ([0, 0, 0, 0], 0)
    whole = lib.exodus_hbm_alloc_striped(size, 0, None)
    assert whole == base
    lib.exodus_hbm_free(whole, size, 0, None)
    e = lib.exodus_hbm_alloc_region1(MIB, 0, None)            # no such range: ordinary memory
    assert e and not base <= e < base + size and usage()[1] == MIB
    assert regions.close() is True                             # what lies elsewhere does not hold the ranges
    assert usage() == ([0, 0, 0, 0], MIB)
    lib.exodus_hbm_free(e, MIB, 0, None)
    assert usage() == ([0, 0, 0, 0], 0)


class _Bytes:
    def __init__(self, ptr, nbytes):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "version": 2, "data": (ptr, False)}


def test_bound_on_what_the_set_up_may_hold(hbm):
    """``take_limit_gib``: the set-up holds no more than that much device memory while it works."""
    regions = hbm.HbmRegions(gib_striped=6.0, take_limit_gib=100.0)
    assert regions.report["chunks_examined"] <= 25 and regions.sizes[hbm.STRIPED] == 12 * GIB
    t = regions.empty((2 ** 30,))                              # 4 GiB across 64 pages
    assert regions.pool_of(t) == hbm.STRIPED
    t.copy_(torch.arange(2 ** 30, device=t.device, dtype=torch.int32) % 1024)
    assert t.view(-1, 1024).eq(torch.arange(1024, device=t.device, dtype=torch.float32)).all()
    del t
    assert regions.close() is True
    with pytest.raises(RuntimeError, match="out of memory"):
        hbm.HbmRegions(gib_striped=6.0, take_limit_gib=16.0)   # 15 probe chunks + 3 for the range do not fit 4 chunks
    with pytest.raises(ValueError):
        hbm.HbmRegions(gib_striped=6.0, take_limit_gib=0.0)


def test_ranges_sorted_by_timed_copies(hbm):
    """``sort=True``: ranges of one region each next to the striped one.  Skipped when this machine's free memory no
    longer shows regions (memory that earlier processes allocated in 64 MiB pages comes back as a mixture)."""
    from sinabs.exodus import _hip as hip
    dev = torch.device("cuda:0")
    try:
        regions = hbm.enable(gib_per_region=8.0, gib_striped=12.0)
    except RuntimeError as err:
        if "did not show three kinds" in str(err):
            pytest.skip("device memory comes back mixed from earlier processes: no regions to sort by")
        raise
    print(f"\nset-up {regions.setup_s:.2f} s; {regions.report}")
    assert regions.sorted and regions.report["kinds_found"] == 3
    assert regions.sizes == [8 * GIB] * 3 + [12 * GIB]
    spans = sorted(zip(regions.bases, regions.sizes))
    assert all(spans[k][0] + spans[k][1] <= spans[k + 1][0] for k in range(3))
    t = regions.empty((3, 1000, 1000), region=1)
    assert regions.pool_of(t) == 1 and regions.bytes_in_use(1) == 12 * MIB    # 12e6 bytes rounded up to 2 MiB pieces
    n, steps = 262144, 1024                                    # 1 GiB per tensor
    x = regions.empty((n, steps), region=0).normal_(0.0, 1.0, generator=torch.Generator(device=dev).manual_seed(5))
    alpha = torch.full((n,), 0.9, device=dev)
    zeros = torch.zeros(n, device=dev)
    one_region = regions.empty((n, steps), region=1)
    striped = regions.empty((n, steps))
    assert regions.pool_of(one_region) == 1 and regions.pool_of(striped) == hbm.STRIPED
    hip.leakyForward(x, zeros, alpha, output=one_region)
    hip.leakyForward(x, zeros, alpha, output=striped)
    own = hip.leakyForward(x, zeros, alpha)                    # the wrapper's own allocation: striped
    assert regions.pool_of(own) == hbm.STRIPED and torch.equal(own, striped) and torch.equal(one_region, striped)
    with pytest.raises(ValueError):
        hbm.HbmRegions(gib_per_region=1.0, gib_striped=0.0, sort=False)


def test_too_little_free_memory_is_refused(hbm):
    with pytest.raises(ValueError):
        hbm.HbmRegions(gib_per_region=96.0)
    free, _ = torch.cuda.mem_get_info()
    held = torch.empty(free - 40 * 2 ** 30, dtype=torch.uint8, device="cuda:0")
    with pytest.raises(RuntimeError, match="out of memory"):
        hbm.HbmRegions(gib_striped=24.0)
    del held
    assert hbm.active() is None


def test_environment_switch_stands_for_enable(hbm, monkeypatch):
    """``SINABS_EXODUS_HBM=striped:<GiB>``: a program that never calls ``enable()`` gets the ranges at its first kernel
    output of 64 MiB or more -- not for small layers, not again after ``disable()``, and with a warning instead of an
    error for a value that cannot be read."""
    import sinabs.exodus.layers as el
    dev = torch.device("cuda:0")
    layer = el.IAF().to(dev)
    small = (torch.rand(2, 50, 256, generator=gen(31)) * 0.6).to(dev)
    big = (torch.rand(8, 200, 16384, generator=gen(32)) * 0.6).to(dev)          # 100 MiB per tensor

    def run(x):
        layer.reset_states()
        return layer(x)

    want = run(big)
    monkeypatch.setattr(hbm, "_switch_tried", False)
    monkeypatch.setenv(hbm.ENVIRONMENT_SWITCH, "nonsense:4")
    with pytest.warns(UserWarning, match="no placement"):
        assert torch.equal(run(big), want)
    assert hbm.active() is None and hbm._switch_tried is True
    monkeypatch.setattr(hbm, "_switch_tried", False)
    monkeypatch.setenv(hbm.ENVIRONMENT_SWITCH, "striped:6")
    run(small)
    assert hbm.active() is None                                 # nothing big enough yet
    got = run(big)
    regions = hbm.active()
    assert regions is not None and regions.sizes[hbm.STRIPED] == 12 * GIB
    assert regions.pool_of(got) == hbm.STRIPED and torch.equal(got, want)
    del got
    layer.reset_states()
    gc.collect()
    assert hbm.disable() is True
    again = run(big)
    assert hbm.active() is None and torch.equal(again, want)    # switched off by hand: it stays off
