"""Region-aware allocation (sinabs.exodus.hbm): the three ranges are made of one region of HBM each (checked by
timed copies), the layer wrappers put what they write into another range than what they read, and no result
changes with where the tensors lie.  The reference has no
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


def test_ranges_are_made_of_one_region_each(hbm):
    """Copies between the ranges beat copies inside one range -- the property the placement is for -- whatever
    this process and earlier ones have done to the order in which the driver hands out memory."""
    regions = hbm.enable(gib_per_region=16.0)
    rep = regions.report
    print(f"\n{rep}")
    inside, across = rep["inside_one_range_GBs"], rep["across_ranges_GBs"]
    assert rep["kinds_found"] == 3 and regions.verified is True
    assert sum(across) / 6 > 1.025 * sum(inside) / 3            # what `verified` says
    spans = sorted(zip(regions.bases, regions.sizes))
    assert all(n == 16 * 2 ** 30 for _, n in spans)
    assert all(spans[k][0] + spans[k][1] <= spans[k + 1][0] for k in range(2))
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
    # closing with a live tensor keeps the memory until the tensor goes
    keep = regions.empty((2 ** 20,), region=0).fill_(7.0)
    hbm.disable()
    assert hbm.active() is None and keep.sum().item() == 7 * 2 ** 20
    assert regions.pool_of(regions.empty((2 ** 20,), region=0)) is None
    del keep


def test_outputs_go_to_another_pool_and_results_do_not_change(hbm):
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

    regions = hbm.enable(gib_per_region=8.0)
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


def test_too_little_free_memory_is_refused(hbm):
    with pytest.raises(ValueError):
        hbm.HbmRegions(gib_per_region=96.0)
    free, _ = torch.cuda.mem_get_info()
    held = torch.empty(free - 40 * 2 ** 30, dtype=torch.uint8, device="cuda:0")
    with pytest.raises(RuntimeError, match="out of memory"):
        hbm.HbmRegions(gib_per_region=8.0)
    del held
    assert hbm.active() is None
