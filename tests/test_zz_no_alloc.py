"""``exodus_layer_lif_backward_from_input``: the backward pass of the layer for callers that cannot
allocate device memory.  It takes no checkpoints; it rebuilds them in a fixed array inside the
library's device image and must give exactly what ``exodus_layer_lif_backward`` gives from the
checkpoints the forward pass wrote -- same kernels, same bits.  Calls share the array, so the tests
run several calls in a row, a larger input first and a smaller one after it."""
import ctypes

import pytest
import torch

from _util import gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    assert torch.cuda.is_available()
    from sinabs.exodus import _hip
    return _hip


def case(hip, b, t, m, syn, cap, seed, kind="single", with_last=True, lo=True):
    """Inputs on the device, the forward pass with checkpoints, and both backward passes."""
    g = gen(seed)
    n = b * m
    D = lambda z: None if z is None else z.cuda()
    scale = 0.5 if syn else 0.8
    x = D(torch.randn(b, t, m, generator=g) * scale + 0.3 * scale)
    am = D(0.5 + 0.5 * torch.rand(n, generator=g)); asn = D(0.3 + 0.6 * torch.rand(n, generator=g)) if syn else None
    v0 = D(torch.randn(n, generator=g) * 0.3); i0 = D(torch.randn(n, generator=g) * 0.3) if syn else None
    # subtract value below the threshold: every factor alpha (1 - c ds/dv) of the reverse recurrence stays
    # within [-1, 1], so gradients stay finite over thousands of steps
    th = D(0.5 + torch.rand(n, generator=g)); c = th * D(0.3 + 0.6 * torch.rand(n, generator=g))
    lo_t = D(-0.2 - torch.rand(n, generator=g)) if lo else None
    go = D(torch.randn(b, t, m, generator=g))
    gvl = D(torch.randn(n, generator=g)) if with_last else None
    gil = D(torch.randn(n, generator=g)) if (with_last and syn) else None
    f = hip.layerLifForward(x, v0, i0, am, asn, c, th, lo_t, lo, cap, True, True)
    surr = None
    if kind == "single":
        k, p0, p1 = hip.SURR_SINGLE_EXP, 0.5, 1.0
    elif kind == "heaviside":
        k, p0, p1 = hip.SURR_HEAVISIDE, 0.7, 0.0
    else:
        k, p0, p1 = hip.SURR_TENSOR, 0.0, 0.0
        surr = D(torch.rand(b, t, m, generator=g))
    args = (am, asn, c, th, lo_t, lo, cap, True, True, k, p0, p1)
    want = hip.layerLifBackward(go, gvl, gil, x, f["ckpt_v"], f["ckpt_i"], v0, i0, *args, surr=surr)
    got = hip.layerLifBackward(go, gvl, gil, x, None, None, v0, i0, *args, surr=surr)
    return want, got


def same(want, got, what):
    for k, (w, g) in enumerate(zip(want, got)):
        assert (w is None) == (g is None), f"{what}: output {k}"
        if w is not None:
            assert bool(torch.isfinite(w).all()), f"{what}: output {k} of exodus_layer_lif_backward is not finite"
            assert torch.equal(w, g), f"{what}: output {k} differs from exodus_layer_lif_backward"
    assert bool(torch.isfinite(got[0]).all()) and bool((got[0] != 0).any()), what


def test_two_calls_in_a_row_the_second_smaller(hip):
    """The second call finds the first call's checkpoints in the array and must not be misled by them."""
    for rep in range(2):
        same(*case(hip, 4, 200, 1024, True, 2, 1), f"large, synaptic (round {rep})")
        same(*case(hip, 2, 70, 96, True, 2, 2), f"small after large, synaptic (round {rep})")
        same(*case(hip, 3, 97, 1000, False, 1, 3), f"no synapse, ragged width (round {rep})")
        same(*case(hip, 1, 1, 1, False, -1, 4, with_last=False, lo=False), f"one neuron, one step (round {rep})")


@pytest.mark.parametrize("kind", ["heaviside", "tensor"])
@pytest.mark.parametrize("t", [31, 32, 33, 129])
def test_other_surrogates_and_sequence_ends(hip, kind, t):
    same(*case(hip, 2, t, 260, True, -1, 10 + t, kind=kind), f"{kind}, {t} steps")
    same(*case(hip, 3, t, 7, False, 3, 20 + t, kind=kind), f"{kind}, {t} steps, 7 neurons")


def test_batch_walked_in_slices_when_the_array_holds_fewer_elements(hip):
    """(5, 2048, 65536) with synapse: one batch element needs 2 x 64 x 65536 floats = half the array, so
    the call walks the batch in slices of two, two and one element, reusing the array each time."""
    free, _ = torch.cuda.mem_get_info()
    if free < 24 * 2 ** 30:
        pytest.skip("needs 24 GiB of free device memory")
    b, t, m = 5, 2048, 65536
    assert 2 * (t // hip.checkpointInterval()) * m * 2 == hip.scratchFloats()
    same(*case(hip, b, t, m, True, 2, 7), "sliced batch")
    same(*case(hip, 2, 64, 512, True, 2, 8), "small call after the sliced one")


def test_sizes_beyond_the_array_are_refused(hip):
    b, t, m = 1, 32 * 300, 1 << 16                       # 300 checkpoints of 65536 neurons > 2^24 floats
    x = torch.zeros(b, t, m, device="cuda"); r = torch.ones(m, device="cuda")
    with pytest.raises(hip.ExodusHipError, match="scratch"):
        hip.layerLifBackward(x, None, None, x, None, None, r, None, r, None, r, r, None, False, 1, True, True,
                             hip.SURR_SINGLE_EXP, 0.5, 1.0)
    # the same tensors with caller-allocated checkpoints are fine
    f = hip.layerLifForward(x, r, None, r, None, r, r, None, False, 1, True, True)
    hip.layerLifBackward(x, None, None, x, f["ckpt_v"], None, r, None, r, None, r, r, None, False, 1, True, True,
                         hip.SURR_SINGLE_EXP, 0.5, 1.0)
    torch.cuda.synchronize()


def test_the_call_allocates_nothing(hip):
    """Raw C ABI with every output preallocated: neither torch's allocator nor the device's free memory
    moves across the call (after a first call, which loads the library's device image)."""
    b, t, m = 3, 100, 512
    n = b * m
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(b, t, m, generator=g, device="cuda") * 0.5 + 0.2
    go = torch.randn(b, t, m, generator=g, device="cuda")
    am = torch.full((n,), 0.9, device="cuda"); asn = torch.full((n,), 0.8, device="cuda")
    one = torch.ones(n, device="cuda"); zero = torch.zeros(n, device="cuda")
    outs = [torch.empty(b, t, m, device="cuda")] + [torch.empty(n, device="cuda") for _ in range(4)]
    P = lambda z: None if z is None else ctypes.c_void_p(z.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call():
        rc = hip.lib.exodus_layer_lif_backward_from_input(
            *[P(o) for o in outs], P(go), None, None, P(x), P(zero), P(zero), P(am), P(asn), P(one), P(one), None,
            0, 2, 1, 1, hip.SURR_SINGLE_EXP, 0.5, 1.0, None, None, None, 0, b, t, m, stream)
        assert rc == 0

    call()
    torch.cuda.synchronize()
    first = [o.clone() for o in outs]
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    assert before == after
    assert all(torch.equal(p, q) for p, q in zip(first, outs))
    f = hip.layerLifForward(x, zero, zero, am, asn, one, one, None, False, 2, True, True)
    want = hip.layerLifBackward(go, None, None, x, f["ckpt_v"], f["ckpt_i"], zero, zero, am, asn, one, one, None, False,
                                2, True, True, hip.SURR_SINGLE_EXP, 0.5, 1.0)
    assert all(torch.equal(p, q) for p, q in zip(want, outs))
