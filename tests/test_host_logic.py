"""CPU-only checks: the C-ABI library loads and exports everything the header declares, and the
host-side mirror of the reference API (layers, conversion, argument handling) behaves.  No kernel
is launched here."""
import ctypes
import os
import re
import subprocess

import pytest
import torch
import torch.nn as nn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "exodus_hip.h")
LIB = os.path.join(ROOT, "sinabs-exodus_amd", "sinabs", "exodus", "libexodus_hip.so")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(exodus_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("exodus_lif_forward", "exodus_lif_backward", "exodus_lif_backward_alpha", "exodus_leaky_forward",
                 "exodus_leaky_backward", "exodus_leaky_backward_alpha", "exodus_leaky_backward_fused",
                 "exodus_lif_backward_fused", "exodus_synlif_forward", "exodus_synlif_backward",
                 "exodus_hip_abi_version", "exodus_hip_error_string"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build the library first: python sinabs-exodus_amd/build_hip.py"
    import torch  # noqa: F401  (loads the HIP runtime the library links against)
    lib = ctypes.CDLL(LIB)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in exodus_hip.h but not exported"
    exported = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True).stdout
    extra = [l.split()[-1] for l in exported.splitlines() if " T " in l and not l.split()[-1].startswith("exodus_")]
    assert not extra, f"unexpected exported symbols: {extra}"
    lib.exodus_hip_abi_version.restype = ctypes.c_int
    assert lib.exodus_hip_abi_version() == 8


def test_layer_entry_points_reject_too_wide_layers_before_touching_the_device():
    """Argument checks come first, so this needs no GPU: 2^25 neurons per batch element is beyond the
    32-bit step offsets of the layer-layout kernels."""
    from sinabs.exodus import _hip
    wide = _hip.LAYER_MAX_NEURONS
    null = None
    rc = _hip.lib.exodus_layer_lif_forward(*([null] * 16), 0, -1, 1, 1, 0, 1, 4, wide, null)
    assert rc == 1
    rc = _hip.lib.exodus_layer_leaky_forward(*([null] * 6), 1, 1, 1, 4, wide, null)
    assert rc == 1
    assert _hip.lib.exodus_layer_lif_forward(*([null] * 16), 0, -1, 1, 1, 0, 0, 4, 8, null) == 0   # empty batch


def test_backward_without_allocation_rejects_what_its_scratch_cannot_hold():
    """The size check of exodus_layer_lif_backward_from_input comes before anything touches a device:
    one batch element whose checkpoints exceed the fixed scratch array is refused with the library's
    own status, and the message says what to use instead."""
    from sinabs.exodus import _hip
    cap = _hip.scratchFloats()
    assert cap == 1 << 24
    ck = _hip.checkpointInterval()
    fake = ctypes.c_void_p(4096)                       # never dereferenced: the call returns before any launch
    def call(t, neurons, syn):
        ptrs = [fake] * 16
        if not syn:
            ptrs[10] = None                            # isyn_initial
            ptrs[12] = None                            # alpha_syn
        return _hip.lib.exodus_layer_lif_backward_from_input(*ptrs, 0, -1, 1, 1, _hip.SURR_SINGLE_EXP, 0.5, 1.0,
                                                             None, None, None, 0, 3, t, neurons, None)
    assert call(ck * 1000, 1 << 20, False) == -2       # 1000 checkpoints of 2^20 neurons
    assert call(ck * 16, 1 << 20, True) == -2          # fits once, but not for potential and current
    assert call(ck * 16 + 1, 1 << 20, False) == -2     # one step more needs one checkpoint more
    msg = _hip.lib.exodus_hip_error_string(-2).decode()
    assert "scratch" in msg and "exodus_layer_lif_backward" in msg
    with pytest.raises(_hip.ExodusHipError, match="scratch"):
        _hip._check(-2, "exodus_layer_lif_backward_from_input")
    assert _hip.lib.exodus_layer_lif_backward_from_input(*([fake] * 16), 0, -1, 1, 1, 9, 0.5, 1.0, None, None, None,
                                                         0, 1, 8, 8, None) == 1  # unknown surrogate kind
    assert _hip.lib.exodus_layer_lif_backward_from_input(*([None] * 16), 0, -1, 1, 1, 1, 0.5, 1.0, None, None, None,
                                                         0, 0, 8, 8, None) == 0  # empty batch
    # one value as the gradient of every spike: not with a surrogate read from a tensor, nor with gradients on records
    assert _hip.lib.exodus_layer_lif_backward_from_input(*([fake] * 16), 0, -1, 1, 1, _hip.SURR_TENSOR, 0.5, 1.0, fake,
                                                         None, None, 1, 1, 8, 8, None) == 1
    assert _hip.lib.exodus_layer_lif_backward(*([fake] * 18), 0, -1, 1, 1, _hip.SURR_SINGLE_EXP, 0.5, 1.0, None, fake,
                                              fake, 1, 1, 8, 8, None) == 1


def test_loader_signatures_cover_the_header():
    from sinabs.exodus import _hip
    assert sorted(_hip._SIGNATURES) == declared_functions()


def test_functions_reject_cpu_tensors_and_bad_arguments():
    from sinabs.exodus.leaky import LeakyIntegrator
    from sinabs.exodus.spike import IntegrateAndFire, classify_surrogate
    from sinabs.exodus._compat import activation as act
    from sinabs.exodus import _hip

    x = torch.rand(2, 10); r = torch.full((2,), 0.5)
    with pytest.raises(RuntimeError, match="no CPU path"):
        LeakyIntegrator.apply(x, r, r)
    with pytest.raises(ValueError, match="2D"):
        LeakyIntegrator.apply(x[0], r, r)
    with pytest.raises(ValueError, match="contiguous"):
        LeakyIntegrator.apply(torch.rand(10, 2).t(), r, r)
    with pytest.raises(ValueError, match="1D"):
        LeakyIntegrator.apply(x, r.unsqueeze(0), r)
    with pytest.raises(ValueError, match="between 0 and 1"):
        IntegrateAndFire.apply(x, torch.tensor([0.5, 1.5]), r, r, r, None, act.Heaviside())
    with pytest.raises(ValueError, match="greater than `min_v_mem`"):
        IntegrateAndFire.apply(x, r, r, torch.ones(2), None, torch.tensor([1.2, 0.0]), act.Heaviside())
    with pytest.raises(RuntimeError, match="no CPU path"):
        IntegrateAndFire.apply(x, r, r, torch.ones(2), None, None, act.Heaviside())

    assert classify_surrogate(act.SingleExponential(0.3, 2.0)) == (_hip.SURR_SINGLE_EXP, 0.3, 2.0)
    assert classify_surrogate(act.PeriodicExponential())[0] == _hip.SURR_PERIODIC_EXP
    assert classify_surrogate(act.Heaviside(0.7)) == (_hip.SURR_HEAVISIDE, 0.7, 0.0)
    assert classify_surrogate(lambda v, th: v)[0] == _hip.SURR_TENSOR

    class SingleExponential:           # same name, foreign module: must not be mistaken for the known one
        grad_width, grad_scale = 0.5, 1.0

    assert classify_surrogate(SingleExponential())[0] == _hip.SURR_TENSOR


def test_layer_construction_and_bookkeeping():
    import sinabs.exodus.layers as el
    from sinabs.exodus._compat import activation as act
    from sinabs.exodus.layers.lif import expand_to_1d_contiguous

    lif = el.LIF(tau_mem=20.0, tau_syn=5.0, min_v_mem=-1.0, train_alphas=True, spike_fn=act.MaxSpike(2))
    assert lif.does_spike and lif.max_num_spikes_per_bin == 2 and lif.decay_early
    assert "EXODUS" in repr(lif)
    assert set(lif.state_dict()) == {"alpha_mem", "alpha_syn", "spike_threshold", "min_v_mem", "v_mem", "i_syn"}
    assert torch.allclose(lif.alpha_mem_calculated, torch.exp(torch.tensor(-1 / 20.0)))
    assert el.LIF(tau_mem=20.0, spike_fn=act.SingleSpike).max_num_spikes_per_bin == 1
    assert el.LIF(tau_mem=20.0).max_num_spikes_per_bin is None
    assert set(el.LIF(tau_mem=20.0).state_dict()) == {"tau_mem", "spike_threshold", "v_mem"}

    iaf = el.IAF(min_v_mem=-2)
    assert iaf.tau_mem is None and float(iaf.alpha_mem_calculated) == 1.0 and not iaf.norm_input
    assert "tau_mem" not in iaf.arg_dict and "norm_input" not in iaf.arg_dict
    leak = el.ExpLeak(tau_mem=10.0)
    assert not leak.does_spike and not leak.decay_early and "spike_fn" not in leak.arg_dict
    sq = el.IAFSqueeze(batch_size=12, min_v_mem=-1)
    assert sq.arg_dict["batch_size"] == 12 and sq.arg_dict["num_timesteps"] == -1
    with pytest.raises(TypeError):
        el.LIFSqueeze(tau_mem=10.0)

    with pytest.raises(NotImplementedError):
        el.LIF(tau_mem=20.0, reset_fn=act.MembraneReset())
    with pytest.raises(NotImplementedError):
        el.IAF(spike_fn=torch.relu)

    lif.reset_states()                                   # uninitialised: a no-op
    lif.init_state_with_shape((3, 4))
    assert lif.is_state_initialised() and lif.state_has_shape((3, 4)) and not lif.state_has_shape((4, 3))
    lif.v_mem += 1.0
    lif.reset_states()
    assert (lif.v_mem == 0).all()

    e = expand_to_1d_contiguous(torch.tensor([1.0, 2.0, 3.0]), (2, 3))
    assert e.tolist() == [1, 2, 3, 1, 2, 3] and e.is_contiguous()
    assert expand_to_1d_contiguous(0.5, (2, 2)).tolist() == [0.5] * 4


def _model(layers_mod, batch_size=12):
    return nn.Sequential(
        nn.Conv2d(2, 8, 5, 1),
        layers_mod.IAFSqueeze(batch_size=batch_size, min_v_mem=-1),
        nn.AvgPool2d(2, 2),
        nn.Conv2d(8, 16, 3, 1),
        layers_mod.IAFSqueeze(batch_size=batch_size, min_v_mem=-2),
        nn.AvgPool2d(2, 2),
        nn.Flatten(),
        nn.Linear(64, 10),
    )


def test_conversion_both_ways():
    """reference tests/test_conversion.py, with the oracle's plain layers in the role of sinabs.layers"""
    import sinabs.exodus.layers as el
    from sinabs.exodus import conversion
    from oracle import sinabs_layers as sl

    plain = _model(sl)
    fast = conversion.sinabs_to_exodus(plain, sinabs_layers=sl)
    assert type(plain[1]) is sl.IAFSqueeze and type(fast[1]) is el.IAFSqueeze and len(plain) == len(fast)
    assert fast[1].min_v_mem == plain[1].min_v_mem and fast[4].min_v_mem == plain[4].min_v_mem
    assert fast[1].batch_size == plain[1].batch_size
    assert torch.equal(fast[0].weight, plain[0].weight) and fast[0] is not plain[0]

    fast2 = _model(el)
    plain2 = conversion.exodus_to_sinabs(fast2, sinabs_layers=sl)
    assert type(plain2[1]) is sl.IAFSqueeze and type(fast2[1]) is el.IAFSqueeze and len(plain2) == len(fast2)
    assert plain2[4].min_v_mem == fast2[4].min_v_mem and plain2[1].batch_size == fast2[1].batch_size

    assert set(conversion.get_module_map(sl).values()) == {el.IAF, el.IAFSqueeze, el.LIF, el.LIFSqueeze, el.ExpLeak,
                                                           el.ExpLeakSqueeze}
    from sinabs.exodus._compat import HAVE_UPSTREAM_SINABS
    if not HAVE_UPSTREAM_SINABS:
        with pytest.raises(ImportError, match="sinabs"):
            conversion.sinabs_to_exodus(plain)


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run(["python", os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0 and "one GPU" in (out.stderr + out.stdout)


def test_bench_placement_modes_choose_the_ranges():
    """bench.py's Placement: where each kind of tensor (0 = read, 1 / 2 = written) is asked from in every mode, and
    that the roofline's traffic figures name a committed profile."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)

    class Ranges:
        sorted, verified, setup_s = True, True, 1.234
        report = {"chunks_examined": 70, "inside_one_range_GBs": [5900.4, 6000.0, 6100.0]}

        def empty(self, shape, region=None):
            return ("range", region, tuple(shape))

    def asked(mode, k):
        got = bench.Placement(torch, "cpu", Ranges(), mode=mode).empty((2, 3), k)
        return "ordinary" if isinstance(got, torch.Tensor) else got[1]

    assert [asked("striped", k) for k in (0, 1, 2)] == ["ordinary", None, None]   # None: the striped range
    assert [asked("all-striped", k) for k in (0, 1, 2)] == [None, None, None]
    assert [asked("regions", k) for k in (0, 1, 2)] == [0, 1, 2]
    assert [asked("one-region", k) for k in (0, 1, 2)] == [0, 0, 0]
    plain = bench.Placement(torch, "cpu")
    assert plain.empty((2, 3), 1).shape == (2, 3) and plain.describe() == {"placement": "ordinary allocator"}
    d = bench.Placement(torch, "cpu", Ranges(), mode="striped").describe()
    assert "alternate" in d["placement"] and d["placement_setup_s"] == 1.234
    assert d["placement_measured"]["inside_one_range_GBs"] == [5900, 6000, 6100] and d["placement_verified_by_timed_copies"]
    assert bench.MEASURED_TRAFFIC, "profiles/traffic.json is missing or empty"
    for (_, _), (nbytes, source) in bench.MEASURED_TRAFFIC.items():
        assert nbytes > 1e9 and source.startswith("profiles/")
        assert os.path.exists(os.path.join(ROOT, source)), source


def test_parameter_validation_modes():
    from sinabs.exodus import _validate as val
    good, bad = torch.tensor([0.0, 0.5, 1.0]), torch.tensor([0.5, 1.5])
    th, lo_ok, lo_bad = torch.ones(2), torch.tensor([-1.0, 0.0]), torch.tensor([1.2, 0.0])
    assert val.get_mode() == "sync"
    val.check_parameters([good], th, lo_ok)
    with pytest.raises(ValueError, match="between 0 and 1"):
        val.check_parameters([good, bad])
    with pytest.raises(ValueError, match="greater than `min_v_mem`"):
        val.check_parameters([good], th, lo_bad)
    try:
        val.set_mode("off")
        val.check_parameters([bad], th, lo_bad)               # nothing is checked
        val.set_mode("deferred")
        with pytest.raises(ValueError):                          # CPU tensors cannot be deferred: raised at once
            val.check_parameters([bad])
        with pytest.raises(ValueError):
            val.set_mode("nonsense")
    finally:
        val.set_mode("sync")


def test_hbm_argument_checks_and_sorting_retries_without_a_device():
    """Argument checks of sinabs.exodus.hbm, and the second try with finer pieces when the big ones show no regions."""
    from sinabs.exodus import hbm
    MIB = 2 ** 20
    for bad in (dict(gib_per_region=-1.0), dict(gib_per_region=0.0, gib_striped=0.0), dict(gib_per_region=70.0, gib_striped=48.0),
                dict(gib_per_region=1.0, sort=False), dict(chunk_bytes=100 * MIB), dict(take_limit_gib=-2.0)):
        with pytest.raises((ValueError, RuntimeError)):      # RuntimeError: no device in this process
            hbm.HbmRegions(**bad)
    # the environment's way of asking for enable()
    assert hbm._read_switch("") is None and hbm._read_switch(" off ") is None
    assert hbm._read_switch("striped") == (48.0, False) and hbm._read_switch("Striped:72") == (72.0, False)
    assert hbm._read_switch("everything:12.5") == (12.5, True) and hbm._read_switch("on") == (48.0, False)
    for bad in ("bogus", "striped:x", "striped:-1", "everything:0"):
        with pytest.raises(ValueError):
            hbm._read_switch(bad)
    # sorting is tried again with finer pieces when the big ones show no regions
    class Lib:
        def __init__(self, outcomes):
            self.outcomes, self.calls, self.destroyed = list(outcomes), [], 0

        def exodus_hbm_regions_create(self, dev, per_region, striped, chunk, sort, take_limit, rep_ref):
            self.calls.append(chunk)
            rc, kinds = self.outcomes.pop(0)
            rep_ref._obj.kinds_found = kinds
            return rc

        def exodus_hbm_regions_destroy(self, dev):
            self.destroyed += 1
            return 0

    sizes = [4096 * MIB, 256 * MIB]
    lib = Lib([(0, 3)])
    assert hbm._create(lib, 0, 0, 1, sizes, True)[::2] == (0, 4096 * MIB) and lib.calls == [4096 * MIB]
    lib = Lib([(hbm.REGIONS_NOT_FOUND, 2), (0, 3)])
    rc, rep, size = hbm._create(lib, 0, 1, 1, sizes, True)
    assert (rc, rep.kinds_found, size) == (0, 3, 256 * MIB) and lib.destroyed == 0
    lib = Lib([(0, 2), (0, 1)])                                   # a striped range alone, unsorted both times
    rc, rep, size = hbm._create(lib, 0, 0, 1, sizes, True)
    assert (rc, rep.kinds_found, size) == (0, 1, 256 * MIB) and lib.destroyed == 1
    lib = Lib([(2, 0)])                                           # any other error ends the tries
    assert hbm._create(lib, 0, 1, 1, sizes, True)[0] == 2 and lib.calls == [4096 * MIB]
    lib = Lib([(0, 0)])
    assert hbm._create(lib, 0, 0, 1, sizes[:1], False)[::2] == (0, 4096 * MIB)   # no sorting asked for: one call
    assert hbm.active() is None
    like = torch.zeros(4, 5)
    assert hbm.empty_like(like).shape == like.shape and hbm.empty((2, 3), like).shape == (2, 3)   # not enabled: torch's
