#!/usr/bin/env python3
"""Benchmark of the EXODUS neuron-dynamics path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c2|c3|c1] [--no-cpu-baseline]

One "step" is one forward + backward pass of the hot path over one batch of synthetic input that
already lives in HBM, called through the C ABI of libexodus_hip.so with preallocated outputs.
Prints ONE JSON line: neuron-timesteps/s (rows * time steps / wall time of fwd+bwd), the HBM
roofline of the slowest kernel (algorithmic bytes / its mean duration, measured with events on
the launch stream) and a CPU baseline (the sinabs-style per-time-step torch loop with autograd,
timed on this machine's host cores on a bounded sample of the same workload).  Under "others" the
same line carries the other configurations, the (rows, time) kernels, and every configuration
through the public layer API (``sinabs.exodus.layers``: autograd, outputs allocated per call),
each with the figures of the ordinary allocator beside those of ``sinabs.exodus.hbm.enable()``.
"""
import argparse
import contextlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "sinabs-exodus_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# Workloads (the synthetic configurations of the baseline description).  bytes = algorithmic
# fp32 traffic per neuron-timestep of (forward kernel, backward kernel).
WORKLOADS = {
    # LIF with synaptic current: tau_syn=5 -> tau_mem=20, min_v_mem=-1, <=2 spikes/step, trainable alphas
    "c5": dict(name="C5 synaptic LIF fwd+bwd (B=16,T=2000,N=65536; tau_syn=5,tau_mem=20,min_v_mem=-1,cap=2,train_alphas)",
               batch=16, steps=2000, neurons=65536, mean=0.05, std=0.5, bytes=(16, 16)),
    # plain LIF, tau_mem=20, single spike
    "c2": dict(name="C2 LIF fwd+bwd (B=32,T=300,N=131072; tau_mem=20,cap=1)",
               batch=32, steps=300, neurons=131072, mean=0.1, std=0.3, bytes=(12, 12)),
    # ExpLeak with trainable per-channel alpha
    "c3": dict(name="C3 ExpLeak fwd+bwd (B=64,T=1000,N=4096; tau~U[5,50] per channel, train_alphas)",
               batch=64, steps=1000, neurons=4096, mean=0.0, std=1.0, bytes=(8, 12)),
    # small IAF
    "c1": dict(name="C1 IAF fwd+bwd (B=8,T=100,N=256; U[0,0.5] input)",
               batch=8, steps=100, neurons=256, mean=None, std=None, bytes=(12, 12)),
}

# HBM traffic per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters
# read for a plain elementwise kernel over exactly 1 GiB in the same runs: bytes per launch by (workload, entry
# point), and the committed summary each figure comes from.  bench_profile.py writes the file from the raw counter
# output when it writes a summary, so the figures cannot drift from the summaries; a kernel that changes needs its
# counters taken again.
def load_measured_traffic():
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            raw = json.load(f)
    except (OSError, ValueError):
        return {}
    return {(e["workload"], e["entry_point"]): (float(e["bytes_per_launch"]), e["source"]) for e in raw["kernels"]}


MEASURED_TRAFFIC = load_measured_traffic()

# what the default run reports next to its headline workload: (workload, path)
OTHERS = [("c2", "layer"), ("c3", "layer"), ("c5", "rows"), ("c2", "rows"), ("c3", "rows")]
# ... and through the public layer API: (workload, loss)
# loss: "dense" = out.backward(gradient tensor); "sum" = out.sum().backward(), torch's own reduction over the output;
# "total" = the same loss taken from the layer: firing_rate * numel, i.e. the total the forward kernel counted anyway
API_RUNS = [("c5", "dense"), ("c5", "sum"), ("c5", "total"), ("c2", "dense"), ("c2", "sum"), ("c2", "total"),
            ("c3", "dense"), ("c3", "sum")]


class Placement:
    """Where a workload's tensors are allocated (``mode``; ``regions`` = sinabs.exodus.hbm.HbmRegions):
    striped      what a program gets that calls ``hbm.enable()`` and nothing else: its own inputs (x, grad_output) from
                 the ordinary allocator, everything the kernels write in the striped range, whose 64 MiB pages
                 alternate between the three regions of HBM
    all-striped  every big tensor in the striped range (``hbm.enable(everything=True)``, or layers behind other layers)
    regions      (needs sorted ranges) every tensor in one region's range: inputs in the first, outputs in the second
                 and third
    one-region   (needs sorted ranges) the control: every big tensor in the first region's range
    plain        torch's ordinary allocator"""

    def __init__(self, torch, dev, regions=None, mode="plain"):
        self.torch, self.dev, self.regions, self.mode = torch, dev, regions, mode

    def empty(self, shape, k):
        """k = 0: a tensor the kernels read (input, incoming gradient); 1, 2: tensors they write"""
        if self.regions is None or (self.mode == "striped" and k == 0):
            return self.torch.empty(tuple(shape), device=self.dev)
        if self.mode in ("striped", "all-striped"):
            return self.regions.empty(shape)
        return self.regions.empty(shape, region=0 if self.mode == "one-region" else k)

    def describe(self):
        if self.regions is None:
            return {"placement": "ordinary allocator"}
        text = {"striped": "sinabs.exodus.hbm.enable(): inputs from the ordinary allocator, everything the kernels write in "
                           "memory whose 64 MiB pages alternate between the three regions of HBM",
                "all-striped": "every big tensor in memory whose 64 MiB pages alternate between the three regions of HBM",
                "one-region": "all big tensors in ONE region of HBM (the control experiment)",
                "regions": "one region of HBM per tensor: inputs in the first, outputs in the second and third"}
        out = {"placement": text[self.mode], "placement_setup_s": round(self.regions.setup_s, 3),
               "placement_setup_seconds_taking_sorting_building_checking":
                   self.regions.report.get("seconds_taking_sorting_building_checking"),
               "placement_sorted_by_timed_copies": bool(self.regions.sorted)}
        if self.regions.sorted:
            out["placement_verified_by_timed_copies"] = bool(self.regions.verified)
            out["placement_measured"] = {k: ([round(x) for x in v] if isinstance(v, list) else round(v))
                                         for k, v in self.regions.report.items()}
        return out


SURROGATE = "single"      # --surrogate: which of the surrogate gradients evaluated inside the kernels the workloads use


def chosen_surrogate(hip, act):
    """(kind, p0, p1) as the kernels take them; SingleExponential is what every configuration names."""
    if SURROGATE == "periodic":
        fn = act.PeriodicExponential()
        return hip.SURR_PERIODIC_EXP, fn.grad_width, fn.grad_scale
    if SURROGATE == "heaviside":
        return hip.SURR_HEAVISIDE, act.Heaviside().window, 1.0
    fn = act.SingleExponential()
    return hip.SURR_SINGLE_EXP, fn.grad_width, fn.grad_scale


def build_layer_workload(key, torch, hip, act, dev, place=None, one_value=False):
    """The same workloads on the layer's own (batch, time, neurons) layout: one kernel per direction,
    forward keeps checkpoints only, backward re-reads the input and rebuilds v_mem / i_syn.
    Algorithmic bytes per neuron-timestep: forward 8 (x in, spikes out), backward 12 (grad_spikes
    and x in, grad_x out) -- or 8 with ``one_value``: the gradient of every output element is one number (what a
    sum as the loss hands back), passed as such."""
    w = WORKLOADS[key]
    place = place or Placement(torch, dev)
    B, T, M = w["batch"], w["steps"], w["neurons"]
    N = B * M
    g = torch.Generator(device=dev).manual_seed(list(WORKLOADS).index(key))
    rx, rgo, rs, rgi = 0, 0, 1, 1                  # tensors the kernels read: 0; tensors they write: 1
    x = place.empty((B, T, M), rx)
    x.uniform_(0.0, 0.5, generator=g) if key == "c1" else x.normal_(w["mean"], w["std"], generator=g)
    go = torch.ones(1, device=dev) if one_value else place.empty((B, T, M), rgo).fill_(1.0)
    bwd_bytes = 8 if one_value else 12
    rows = lambda v: torch.as_tensor(v, dtype=torch.float32, device=dev).expand(B, M).flatten().contiguous()
    zeros = torch.zeros(N, device=dev); ones = torch.ones(N, device=dev)
    kind, p0, p1 = chosen_surrogate(hip, act)
    spikes = place.empty(x.shape, rs); gi = place.empty(x.shape, rgi)
    if key == "c5":
        cfg = dict(a_mem=rows(math.exp(-1 / 20.0)), a_syn=rows(math.exp(-1 / 5.0)), lo=rows(-1.0), cap=2, norm=True)
    elif key == "c2":
        cfg = dict(a_mem=rows(math.exp(-1 / 20.0)), a_syn=None, lo=None, cap=1, norm=True)
    elif key == "c1":
        cfg = dict(a_mem=ones, a_syn=None, lo=None, cap=-1, norm=False)
    else:
        # C3: ExpLeak with trainable per-channel alpha; forward 8 B (x in, out out), backward 12 B
        # (grad_out and saved out in, grad_x out)
        tau = 5.0 + 45.0 * torch.rand(M, generator=g, device=dev)
        a_mem = rows(torch.exp(-1.0 / tau))
        holder = {}

        def fwd():
            holder["out"] = hip.layerLeakyForward(x, zeros, a_mem, False, False)[0]

        def bwd():
            r = hip.layerLeakyBackward(go, None, holder["out"], x, zeros, a_mem, False, False, True,
                                       shape=(B, T, M) if one_value else None)
            return r[1].view(B, M).sum(0)

        return dict(fwd=fwd, bwd=bwd, N=N, T=T, fwd_name="exodus_layer_leaky_forward",
                    bwd_name="exodus_layer_leaky_backward", bytes=(8, bwd_bytes))
    syn = cfg["a_syn"] is not None
    holder = {}

    def fwd():
        holder["r"] = hip.layerLifForward(x, zeros, zeros if syn else None, cfg["a_mem"], cfg["a_syn"], ones, ones,
                                          cfg["lo"], cfg["lo"] is not None, cfg["cap"], True, cfg["norm"],
                                          outSpikes=spikes)

    def bwd():
        r = holder["r"]
        out = hip.layerLifBackward(go, None, None, x, r["ckpt_v"], r["ckpt_i"], zeros, zeros if syn else None,
                                   cfg["a_mem"], cfg["a_syn"], ones, ones, cfg["lo"], cfg["lo"] is not None,
                                   cfg["cap"], True, cfg["norm"], kind, p0, p1, gradInput=gi, gradUniform=one_value)
        return out[1].view(B, M).sum(0)

    return dict(fwd=fwd, bwd=bwd, N=N, T=T, fwd_name="exodus_layer_lif_forward",
                bwd_name="exodus_layer_lif_backward", bytes=(8, bwd_bytes))


def build_workload(key, torch, hip, act, dev, place=None):
    w = WORKLOADS[key]
    place = place or Placement(torch, dev)
    B, T, M = w["batch"], w["steps"], w["neurons"]
    N = B * M
    g = torch.Generator(device=dev).manual_seed(list(WORKLOADS).index(key))
    x = place.empty((N, T), 0)
    x.uniform_(0.0, 0.5, generator=g) if key == "c1" else x.normal_(w["mean"], w["std"], generator=g)
    go = place.empty((N, T), 0).fill_(1.0)
    rows = lambda v: torch.as_tensor(v, dtype=torch.float32, device=dev).expand(B, M).flatten().contiguous()
    zeros = torch.zeros(N, device=dev)
    ones = torch.ones(N, device=dev)
    kind, p0, p1 = chosen_surrogate(hip, act)
    fwd_name = bwd_name = None

    if key == "c5":
        a_mem = rows(math.exp(-1 / 20.0)); a_syn = rows(math.exp(-1 / 5.0)); lo = rows(-1.0)
        # the backward kernel reads one tensor from each region and writes into the third; with its three inputs
        # in one region it measured 15 % slower
        s = place.empty(x.shape, 1); v = place.empty(x.shape, 1)
        i = place.empty(x.shape, 2); gi = place.empty(x.shape, 2)

        def fwd():
            hip.synLifForward(x, zeros, zeros, a_mem, a_syn, ones, ones, lo, True, 2, True, True, out=(s, v, i))

        def bwd():
            r = hip.synLifBackward(go, None, None, v, i, zeros, zeros, a_mem, a_syn, ones, ones, lo, True, 2, True,
                                   True, kind, p0, p1, inputGrad=gi)
            # per-row alpha gradients -> per-neuron (what autograd's expand backward does)
            return r[1].view(B, M).sum(0), r[2].view(B, M).sum(0)

        fwd_name, bwd_name = "exodus_synlif_forward", "exodus_synlif_backward"
    elif key in ("c2", "c1"):
        a_mem = rows(math.exp(-1 / 20.0)) if key == "c2" else ones
        cap = 1 if key == "c2" else -1
        xin = x
        if key == "c2":
            xin = place.empty(x.shape, 0)
            torch.mul((1.0 - a_mem).unsqueeze(1), x, out=xin)     # norm_input scaling, done once outside the step
        s = place.empty(x.shape, 1); v = place.empty(x.shape, 1)
        gi = place.empty(x.shape, 2)

        def fwd():
            hip.lifForward(s, v, xin, zeros, a_mem, ones, ones, None, False, cap)

        def bwd():
            return hip.lifBackwardFused(go, None, v, None, a_mem, ones, ones, None, False, cap, kind, p0, p1,
                                        inputGrad=gi)

        fwd_name, bwd_name = "exodus_lif_forward", "exodus_lif_backward_fused"
    elif key == "c3":
        tau = 5.0 + 45.0 * torch.rand(M, generator=g, device=dev)
        a_mem = rows(torch.exp(-1.0 / tau))
        out = place.empty(x.shape, 1)
        gi = place.empty(x.shape, 2)
        holder = {}

        def fwd():
            holder["out"] = hip.leakyForward(x, zeros, a_mem, output=out)

        def bwd():
            r = hip.leakyBackwardFused(go, a_mem, output=holder["out"], vmemInitial=zeros, needAlphaGrad=True,
                                       inputGrad=gi)
            return r[1].view(B, M).sum(0)

        fwd_name, bwd_name = "exodus_leaky_forward", "exodus_leaky_backward_fused"
    return dict(fwd=fwd, bwd=bwd, N=N, T=T, fwd_name=fwd_name, bwd_name=bwd_name)


def cpu_baseline(key, torch, budget_s=12.0):
    """The sinabs-style CPU path (per-step torch ops + autograd BPTT) on a row sample of the workload."""
    from oracle import exodus_ref as ref
    from oracle import sinabs_cpu as sc

    w = WORKLOADS[key]
    T = w["steps"]
    threads = torch.get_num_threads()
    surr = ref.SingleExponential()

    def run(m):
        g = torch.Generator().manual_seed(0)
        if key == "c1":
            x = torch.rand(1, T, m, generator=g) * 0.5
        else:
            x = torch.randn(1, T, m, generator=g) * w["std"] + w["mean"]
        x.requires_grad_(True)
        t0 = time.perf_counter()
        if key == "c5":
            a_m = torch.full((m,), math.exp(-1 / 20.0), requires_grad=True)
            a_s = torch.full((m,), math.exp(-1 / 5.0), requires_grad=True)
            out, _, _ = sc.lif_forward(x, a_m, a_s, {"v_mem": torch.zeros(1, m), "i_syn": torch.zeros(1, m)}, 1.0,
                                       None, surr, 2, -1.0, True)
        elif key == "c2":
            a_m = torch.full((m,), math.exp(-1 / 20.0))
            out, _, _ = sc.lif_forward(x, a_m, None, {"v_mem": torch.zeros(1, m)}, 1.0, None, surr, 1, None, True)
        elif key == "c1":
            out, _, _ = sc.lif_forward(x, torch.tensor(1.0), None, {"v_mem": torch.zeros(1, m)}, 1.0, None, surr,
                                       None, None, False)
        else:
            a_m = torch.exp(-1.0 / (5.0 + 45.0 * torch.rand(m, generator=g))).requires_grad_(True)
            out, _, _ = sc.lif_forward(x, a_m, None, {"v_mem": torch.zeros(1, m)}, None, None, None, None, None,
                                       False, spiking=False)
        out.sum().backward()
        dt = time.perf_counter() - t0
        alphas = a_m if key != "c1" else None
        return dt, x, out.detach(), x.grad, alphas

    m = min(w["batch"] * w["neurons"], 4096)
    run(min(m, 256))                       # warm-up of the op dispatch paths
    res = run(m)
    total = w["batch"] * w["neurons"]
    while res[0] < budget_s / 4 and m < total and m * T * 4 * 40 < 48e9:   # keep the autograd tape under ~48 GB
        m = min(total, m * 4)
        res = run(m)
    dt = res[0]
    return dict(value=m * T / dt, unit="neuron-timesteps/s", cores=threads, kind="port",
                sample=f"{m} of {total} rows x {T} steps, one fwd+bwd in {dt:.2f} s "
                       f"(per-step torch loop + autograd, {threads} threads)",
                parity_on_sample=parity_on_sample(key, torch, m, *res[1:]))


def parity_on_sample(key, torch, m, x, out_cpu, grad_cpu, alphas):
    """The kernels on the very rows the CPU loop just processed (grad_output = ones): fraction of rows
    whose spike trains differ (the CPU loop rounds the synapse update in another order, so a potential
    within rounding distance of the threshold can fall on the other side, after which the row
    legitimately diverges) and the largest gradient error over the rows that agree."""
    from sinabs.exodus import _hip as hip
    dev = torch.device("cuda:0")
    xd = x.detach().to(dev).contiguous()
    full = lambda v: torch.full((m,), float(v), device=dev)
    zeros = torch.zeros(m, device=dev)
    go = torch.ones_like(xd)
    if key == "c3":
        a = alphas.detach().to(dev)
        out, _ = hip.layerLeakyForward(xd, zeros, a, False, False)
        gx = hip.layerLeakyBackward(go, None, out, None, zeros, a, False, False, True)[0]
    else:
        a_m = full(1.0) if key == "c1" else full(math.exp(-1 / 20.0))
        a_s = full(math.exp(-1 / 5.0)) if key == "c5" else None
        lo = full(-1.0) if key == "c5" else None
        cap = {"c5": 2, "c2": 1, "c1": -1}[key]
        norm = key != "c1"
        f = hip.layerLifForward(xd, zeros, zeros if a_s is not None else None, a_m, a_s, full(1.0), full(1.0), lo,
                                lo is not None, cap, True, norm)
        out = f["spikes"]
        gx = hip.layerLifBackward(go, None, None, xd, f["ckpt_v"], f["ckpt_i"], zeros, zeros if a_s is not None else None,
                                  a_m, a_s, full(1.0), full(1.0), lo, lo is not None, cap, True, norm,
                                  hip.SURR_SINGLE_EXP, 0.5, 1.0)[0]
    out = out.cpu()[0].T                                       # (rows, time)
    gx = gx.cpu()[0].T
    want = out_cpu[0].T
    gwant = grad_cpu[0].T
    if key == "c3":
        same = torch.ones(m, dtype=torch.bool)
        out_err = ((out - want).abs() / (1e-5 + 1e-4 * want.abs())).max().item()
    else:
        same = (out == want).all(1)
        out_err = 0.0
    err = ((gx - gwant).abs() / (1e-5 + 1e-4 * gwant.abs()))[same]
    return {"rows": m, "rows_with_differing_spikes": int((~same).sum()), "fraction": float((~same).float().mean()),
            "output_error_in_tolerances": out_err,
            "grad_input_max_abs_error": float((gx - gwant).abs()[same].max()) if same.any() else None,
            "grad_input_error_in_tolerances (rtol 1e-4, atol 1e-5)": float(err.max()) if same.any() else None}


class Probes:
    """ctypes face of libexodus_bench_probes.so: flat streaming kernels (copy / add, read only, write
    only) that only this script uses, as bandwidth yardsticks next to the recurrence kernels."""

    PATH = os.path.join(ROOT, "sinabs-exodus_amd", "libexodus_bench_probes.so")

    def __init__(self, torch):
        import ctypes
        if not os.path.exists(self.PATH):
            raise ImportError(f"{self.PATH} not found; build it with `python sinabs-exodus_amd/build_hip.py`")
        self.torch, self.c = torch, ctypes
        self.lib = ctypes.CDLL(self.PATH)
        p, i64 = ctypes.c_void_p, ctypes.c_int64
        for name, argtypes in (("exodus_probe_stream", [p, p, p, i64, p]), ("exodus_probe_read", [p, i64, p]),
                               ("exodus_probe_write", [p, i64, p])):
            fn = getattr(self.lib, name)
            fn.argtypes, fn.restype = argtypes, ctypes.c_int

    def _call(self, name, *args):
        stream = self.c.c_void_p(self.torch.cuda.current_stream().cuda_stream)
        rc = getattr(self.lib, name)(*args, stream)
        if rc:
            raise RuntimeError(f"{name} failed with hipError {rc}")

    def _ptr(self, x):
        assert x is None or (x.is_cuda and x.dtype == self.torch.float32 and x.is_contiguous())
        return None if x is None else self.c.c_void_p(x.data_ptr())

    def stream(self, dst, a, b=None):
        assert dst.numel() == a.numel() and (b is None or b.numel() == a.numel())
        self._call("exodus_probe_stream", self._ptr(dst), self._ptr(a), self._ptr(b), a.numel())

    def read(self, a):
        self._call("exodus_probe_read", self._ptr(a), a.numel())

    def write(self, dst):
        self._call("exodus_probe_write", self._ptr(dst), dst.numel())


def measure_ceilings(args, torch, hip, dev, place):
    """GB/s of data-movement-only kernels on tensors of the chosen workload's shape, placed as the workload's are
    (what is read as its inputs, what is written as its outputs)."""
    w = WORKLOADS[args.workload]
    B, T, M = w["batch"], w["steps"], w["neurons"]
    n = B * T * M
    a = place.empty((B, T, M), 0).normal_(); b = place.empty((B, T, M), 0).normal_(); out = place.empty((B, T, M), 1)
    alpha = torch.rand(B * M, device=dev) * 0.5 + 0.4
    zeros = torch.zeros(B * M, device=dev)

    def timed(fn):
        for _ in range(max(1, args.warmup)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    res = {"workload": w["name"], "tensor_GB": n * 4 / 1e9, "peak_GBs": HBM_PEAK_GBS, **place.describe()}
    res.pop("placement_measured", None)
    probes = Probes(torch)
    ms = timed(lambda: probes.read(a))
    res["flat_read_only"] = {"ms": ms, "GBs": n * 4 / ms / 1e6}
    ms = timed(lambda: probes.write(out))
    res["flat_write_only"] = {"ms": ms, "GBs": n * 4 / ms / 1e6}
    ms = timed(lambda: probes.stream(out, a))
    res["flat_copy_1r1w"] = {"ms": ms, "GBs": n * 8 / ms / 1e6}
    ms = timed(lambda: probes.stream(out, a, b))
    res["flat_add_2r1w"] = {"ms": ms, "GBs": n * 12 / ms / 1e6}
    ms = timed(lambda: hip.layerLeakyForward(a, zeros, alpha, False, False))
    res["time_strided_1r1w (leaky layer forward)"] = {"ms": ms, "GBs": n * 8 / ms / 1e6}
    ms = timed(lambda: hip.layerLeakyBackward(a, None, b, None, zeros, alpha, False, False, True))
    res["time_strided_2r1w (leaky layer backward with alpha gradient)"] = {"ms": ms, "GBs": n * 12 / ms / 1e6}
    return res


def api_layer(key, torch, dev):
    """The layer of ``sinabs.exodus.layers`` that a configuration names, and the shape of its input."""
    import sinabs.exodus.layers as el
    from sinabs.exodus._compat import activation as act
    if key == "c5":
        layer = el.LIF(tau_mem=20.0, tau_syn=5.0, min_v_mem=-1.0, spike_fn=act.MaxSpike(2), train_alphas=True)
        shape = (16, 2000, 65536)
    elif key == "c2":
        layer = el.LIF(tau_mem=20.0, spike_fn=act.SingleSpike)
        shape = (32, 300, 128, 32, 32)
    elif key == "c3":
        g = torch.Generator().manual_seed(2)
        layer = el.ExpLeak(tau_mem=5.0 + 45.0 * torch.rand(4096, generator=g), train_alphas=True)
        shape = (64, 1000, 4096)
    else:
        layer = el.IAF()
        shape = (8, 100, 256)
    return layer.to(dev), shape


def measure_layer_api(key, loss, torch, dev, steps, warmup, place_all=False):
    """One configuration through the public layer API: ``out = layer(x)`` followed by ``out.backward(grad)`` with a
    dense gradient (``loss == "dense"``) or ``out.sum().backward()`` (``"sum"``): autograd, outputs allocated by every
    call, the layer's state handling and firing rate included.  Wall time per step and the time of each direction
    from events around the two calls.  ``place_all``: the input and the gradient are allocated inside
    ``hbm.placement()`` as well (a layer behind other layers)."""
    from sinabs.exodus import hbm
    w = WORKLOADS[key]
    layer, shape = api_layer(key, torch, dev)
    g = torch.Generator(device=dev).manual_seed(list(WORKLOADS).index(key))
    with (hbm.placement() if place_all else contextlib.nullcontext()):
        x = torch.empty(shape, device=dev)
        x.uniform_(0.0, 0.5, generator=g) if key == "c1" else x.normal_(w["mean"], w["std"], generator=g)
        go = torch.empty(shape, device=dev).uniform_(0.5, 1.5, generator=g) if loss == "dense" else None
    x.requires_grad_(True)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]

    def step(e=None):
        layer.reset_states()
        layer.zero_grad(set_to_none=True)
        x.grad = None
        if e:
            e[0].record()
        out = layer(x)
        if e:
            e[1].record()
        total = None
        if loss == "sum":
            total = out.sum()                                   # torch's own reduction over the output
        elif loss == "total":
            total = layer.firing_rate * float(out.numel())      # the same number, counted by the forward kernel
        if e:
            e[2].record()
        if loss == "dense":
            out.backward(go)
        else:
            total.backward()
        if e:
            e[3].record()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        step(ev[k])
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / steps
    loss_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / steps
    bwd_ms = sum(e[2].elapsed_time(e[3]) for e in ev) / steps
    n_t = 1
    for v in shape:
        n_t *= v
    # bytes that have to move: forward x in, output out (8); backward with a dense gradient: gradient and x in, grad_x
    # out (12); with the sum as the loss the gradient is one value and the backward reads x and writes grad_x (8) --
    # torch's sum over the output (4 more, "loss_ms") is the program's loss, not the layer, and is left out of the fraction
    layer_bytes = 20 if loss == "dense" else 16
    return {"workload": w["name"], "path": "public layer API (sinabs.exodus.layers, autograd, outputs allocated per call)",
            "layer": repr(layer).split("(")[0].strip(), "loss": {"dense": "out.backward(dense gradient)", "sum": "out.sum().backward()",
                     "total": "(layer.firing_rate * out.numel()).backward() -- the sum of the output as the forward kernel "
                              "counted it"}[loss],
            "rows": n_t // shape[1], "time_steps": shape[1], "steps": steps, "ms_per_step": wall * 1e3,
            "fwd_ms": fwd_ms, "loss_ms": loss_ms, "bwd_ms": bwd_ms, "value": n_t / wall, "unit": "neuron-timesteps/s",
            "algorithmic_bytes_per_neuron_timestep": layer_bytes,
            "fwd_bwd_combined_frac": n_t * layer_bytes / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS}


def measure_small_layer(torch, dev, steps, warmup):
    """C1 (8 x 100 x 256, IAF, loss = sum of spikes) through the layer API: one step eagerly, and the same step
    recorded into a HIP graph and replayed (sinabs.exodus.graph.GraphedStep); the two kernels alone from events."""
    from sinabs.exodus.graph import GraphedStep
    import torch.nn as nn
    w = WORKLOADS["c1"]
    layer, shape = api_layer("c1", torch, dev)
    model = nn.Sequential(layer)
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.empty(shape, device=dev).uniform_(0.0, 0.5, generator=g).requires_grad_(True)

    def step():
        layer.reset_states()
        x.grad = None
        out = model(x)
        out.sum().backward()
        return out

    def wall(fn, n):
        for _ in range(max(3, warmup)):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    n = max(200, steps * 10)
    eager_ms = wall(step, n)
    graphed = GraphedStep(model, step)
    replay_ms = wall(graphed.replay, n)
    n_t = shape[0] * shape[1] * shape[2]
    return {"workload": w["name"], "path": "public layer API (sinabs.exodus.layers)", "rows": shape[0] * shape[2],
            "time_steps": shape[1], "steps": n, "ms_per_step_eager": eager_ms, "ms_per_step_hip_graph_replay": replay_ms,
            "value": n_t / (replay_ms * 1e-3), "value_eager": n_t / (eager_ms * 1e-3), "unit": "neuron-timesteps/s"}


def measure_conv_snn(args, torch, dev):
    """Wall clock of one forward + backward of the convolutional spiking network (C4), PyTorch-ROCm for the
    convolution / pooling / linear layers, this package's layers in between; and, from a second run with events
    around every neuron layer's forward and backward pass, the share of the neuron layers."""
    import torch.nn as nn
    import sinabs.exodus.layers as el
    B, T = 64, 300

    def network(neuron):
        layers = [nn.Conv2d(2, 32, 3), neuron(), nn.AvgPool2d(2), nn.Conv2d(32, 64, 3), neuron(), nn.Flatten(),
                  nn.Linear(64 * 14 * 14, 10), neuron()]
        return nn.Sequential(*[l for l in layers if l is not None]).to(dev)

    torch.manual_seed(0)
    x = (torch.rand(B, T, 2, 34, 34, device=dev) < 0.02).float()
    labels = torch.randint(0, 10, (B,), device=dev)

    def make_step(model, spiking=True):
        def step():
            for m in model:
                if hasattr(m, "reset_states"):
                    m.reset_states()
            model.zero_grad()
            out = model(x.flatten(0, 1))
            if spiking:
                loss = nn.functional.cross_entropy(out.reshape(B, T, 10).sum(1), labels)
            else:
                loss = out.sum()
            loss.backward()
        return step

    def timed(step):
        for _ in range(max(1, args.warmup)):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    fast = network(lambda: el.IAFSqueeze(batch_size=B))
    with torch.no_grad():
        for i in (0, 3, 6):
            fast[i].weight.mul_(3.0)                # enough drive for all three layers to spike
    res = {"workload": "C4 conv SNN fwd+bwd (B=64,T=300, 2x34x34 Bernoulli(0.02) input)", "path": "public layer API",
           "neuron_layer_rows": [64 * 32 * 32 * 32, 64 * 64 * 14 * 14, 64 * 10], "time_steps": T, "steps": args.steps}
    res["ms_per_step"] = timed(make_step(fast))
    # the neuron layers' share: events when each layer's forward starts and ends, when the gradient of its output
    # arrives and when the gradient of its input leaves (hooks; they add a little host work, so the end-to-end
    # figure above comes from the run without them)
    spans = []
    handles = []
    for m in fast:
        if not hasattr(m, "reset_states"):
            continue
        ev = {k: torch.cuda.Event(enable_timing=True) for k in ("f0", "f1", "b0", "b1")}
        spans.append(ev)
        handles += [m.register_forward_pre_hook(lambda mod, a, ev=ev: ev["f0"].record()),
                    m.register_forward_hook(lambda mod, a, o, ev=ev: ev["f1"].record()),
                    m.register_full_backward_pre_hook(lambda mod, go, ev=ev: ev["b0"].record()),
                    m.register_full_backward_hook(lambda mod, gi, go, ev=ev: ev["b1"].record())]
    hooked = make_step(fast)
    x.requires_grad_(True)                          # so that the first layer's backward hook has a gradient to wait for
    for _ in range(2):
        hooked()
    total = 0.0
    for _ in range(args.steps):
        hooked()
        torch.cuda.synchronize()
        total += sum(ev["f0"].elapsed_time(ev["f1"]) + ev["b0"].elapsed_time(ev["b1"]) for ev in spans)
    x.requires_grad_(False)
    for h in handles:
        h.remove()
    res["ms_neuron_layers"] = total / args.steps
    for m in fast:
        if hasattr(m, "native_layout"):
            m.native_layout = False
    res["ms_per_step_rows_functions_with_transposes"] = timed(make_step(fast))
    res["ms_conv_pool_linear_alone"] = timed(make_step(network(lambda: None), spiking=False))
    res["value"] = sum(res["neuron_layer_rows"]) * T / (res["ms_per_step"] * 1e-3)
    res["unit"] = "neuron-timesteps/s"
    return res


def measure(wl, steps, warmup, torch):
    """`warmup` untimed and `steps` timed forward + backward passes of a built workload: wall time per
    step and the mean duration of each direction from events on the launch stream."""
    fwd, bwd = wl["fwd"], wl["bwd"]
    for _ in range(warmup):
        fwd(); bwd()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        ev[k][0].record()
        fwd()
        ev[k][1].record()
        bwd()
        ev[k][2].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    f = [e[0].elapsed_time(e[1]) for e in ev]
    b = [e[1].elapsed_time(e[2]) for e in ev]
    return {"steps": steps, "ms_per_step": wall * 1e3 / steps, "fwd_ms": sum(f) / steps, "bwd_ms": sum(b) / steps,
            "fwd_ms_min_max": [min(f), max(f)], "bwd_ms_min_max": [min(b), max(b)]}


def roofline(key, wl, fwd_ms, bwd_ms, bf, bb, traffic_known=True):
    """HBM roofline of the slower of the two kernels: algorithmic bytes per launch / mean duration."""
    n_t = wl["N"] * wl["T"]
    dom = "bwd" if bwd_ms >= fwd_ms else "fwd"
    dom_ms, dom_bytes, dom_name = (bwd_ms, bb, wl["bwd_name"]) if dom == "bwd" else (fwd_ms, bf, wl["fwd_name"])
    other_ms, other_bytes, other_name = (fwd_ms, bf, wl["fwd_name"]) if dom == "bwd" else (bwd_ms, bb, wl["bwd_name"])
    achieved = n_t * dom_bytes / (dom_ms * 1e-3) / 1e9
    traffic, source = MEASURED_TRAFFIC.get((key, dom_name), (None, None)) if traffic_known else (None, None)
    return {
        "bound": "hbm", "kernel": dom_name, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": source,
        "kernel_ms": dom_ms, "algorithmic_bytes_per_launch": n_t * dom_bytes,
        "other_kernel": {"kernel": other_name, "kernel_ms": other_ms,
                         "achieved": n_t * other_bytes / (other_ms * 1e-3) / 1e9},
        "fwd_bwd_combined_frac": n_t * (bf + bb) / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS,
    }


def measure_region_map(args, torch, dev):
    """Rates of a flat copy between every two of the buffers that fill device memory, in allocation order."""
    probes = Probes(torch)
    gib = args.region_map
    nel = int(gib * 2 ** 30) // 4
    free, total = torch.cuda.mem_get_info()
    n = int((free / 2 ** 30 - 6) // gib)
    bufs = [torch.empty(nel, device=dev) for _ in range(n)]
    bufs[0].normal_()

    def rate(dst, src, reps=3):
        probes.stream(dst, src)
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(reps)]
        for a, b in ev:
            a.record(); probes.stream(dst, src); b.record()
        torch.cuda.synchronize()
        return nel * 8 / sorted(a.elapsed_time(b) for a, b in ev)[reps // 2] / 1e6

    mat = [[rate(bufs[j], bufs[i]) if i != j else 0.0 for j in range(n)] for i in range(n)]
    flat = sorted(v for row in mat for v in row if v)
    # the rates fall into two groups; split them at the widest gap between neighbours of the sorted list
    # (looked for between the 10th and the 90th percentile)
    lo, hi = len(flat) // 10, len(flat) * 9 // 10
    cut = max(range(lo, hi), key=lambda k: flat[k + 1] - flat[k])
    threshold = (flat[cut] + flat[cut + 1]) / 2
    for i, row in enumerate(mat):
        print(f"src {i:3d} ({i * gib:5.0f} GiB): " + "".join("-" if i == j else ("#" if v < threshold else ".")
                                                             for j, v in enumerate(row)), flush=True)
    slow_with_first = [j for j in range(1, n) if mat[0][j] < threshold]
    # buffers are grouped by which of them copy slowly into each other
    groups, seen = [], set()
    for i in range(n):
        if i not in seen:
            grp = [i] + [j for j in range(n) if j != i and mat[i][j] < threshold and j not in seen]
            seen.update(grp)
            groups.append(grp)
    inside = [mat[i][j] for g in groups for i in g for j in g if i != j]
    across = [mat[i][j] for a in groups for b in groups if a is not b for i in a for j in b]
    med = lambda r: sorted(r)[len(r) // 2] if r else None
    print(json.dumps({
        "buffers": n, "GiB_each": gib, "device_GiB": total / 2 ** 30, "threshold_GBs": threshold,
        "groups_of_buffers_that_copy_slowly_into_each_other (allocation order, GiB from the first)":
            [[min(g) * gib, (max(g) + 1) * gib, len(g)] for g in groups],
        "copy_inside_one_group_GBs": {"min": min(inside), "median": med(inside), "max": max(inside)},
        "copy_across_groups_GBs": {"min": min(across), "median": med(across), "max": max(across)} if across else None,
        "pairs_on_the_wrong_side_of_the_threshold": sum(v >= threshold for v in inside) + sum(v < threshold for v in across)}))


def child_json(argv, timeout=300):
    """The last line a child run of this script printed, parsed, or {"error": ...}."""
    import subprocess
    try:
        child = subprocess.run([sys.executable, os.path.abspath(__file__)] + argv, capture_output=True, text=True,
                               timeout=timeout)
    except subprocess.TimeoutExpired:
        return {"error": f"no result within {timeout} s"}
    try:
        return json.loads(child.stdout.strip().splitlines()[-1])
    except (IndexError, ValueError):
        return {"error": (child.stderr or child.stdout)[-400:]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c5", choices=list(WORKLOADS))
    ap.add_argument("--path", default="layer", choices=["layer", "rows"],
                    help="layer: kernels on the layer's (batch, time, neurons) layout (what the layers run); "
                         "rows: the (rows, time) kernels behind the autograd Functions")
    ap.add_argument("--shape", default=None, metavar="B,T,M",
                    help="run the chosen workload's layer type and options at another (batch, steps, neurons) shape, "
                         "e.g. a neuron count that does not fill 128-byte memory lines; such a run is a measurement "
                         "aid, not the benchmark (roofline.traffic is then null)")
    ap.add_argument("--one-value-gradient", action="store_true",
                    help="with --path layer: the gradient of every output element is one number, handed to the backward "
                         "kernel as such (what a sum as the loss gives): it reads one tensor less (8 + 8 bytes)")
    ap.add_argument("--surrogate", default="single", choices=["single", "periodic", "heaviside"],
                    help="surrogate gradient of the spiking workloads' kernels (wrappers, --path layer / rows): "
                         "SingleExponential as the configurations name it (default), PeriodicExponential or Heaviside -- "
                         "a measurement aid: the default run and its public-API entries always use SingleExponential")
    ap.add_argument("--one-lane-per-neuron", action="store_true",
                    help="keep the backward kernel that walks a neuron's whole sequence in one lane also for layers with few "
                         "neurons (by default those run the kernel that gives every 32 steps a lane of its own)")
    ap.add_argument("--split-any-size", action="store_true",
                    help="the opposite: run the kernel that gives every 32 steps a lane of its own for layers of any size "
                         "that it can handle (to see where it stops paying; the default draws the line at 16384 neurons)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--others", default="all", choices=["all", "api", "none"],
                    help="all (default): also time the other configurations and the (rows, time) kernels for a few steps "
                         "each, every configuration through the public layer API, the small layer (C1) eagerly and as a "
                         "HIP graph, and the convolutional network (C4), and list them under \"others\"; api: only the "
                         "runs through the public layer API; none: only the chosen workload")
    ap.add_argument("--no-others", dest="others", action="store_const", const="none")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain elementwise kernel (torch.neg) over exactly 1 GiB before the timed region, so that a "
                         "counter run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) has a kernel of known traffic "
                         "to scale its readings by")
    ap.add_argument("--ceilings", action="store_true",
                    help="instead of the benchmark, measure what this machine gives kernels that only move data at the "
                         "default workload's tensor size: a flat copy, a flat 2-read-1-write kernel, and the leaky-"
                         "integrator layer kernels, which walk memory exactly as the spiking kernels do")
    ap.add_argument("--conv-snn", action="store_true",
                    help="instead of the benchmark, time the convolutional configuration end to end through the public "
                         "layer API (Conv2d -> IAFSqueeze -> AvgPool -> Conv2d -> IAFSqueeze -> Flatten -> Linear -> "
                         "IAFSqueeze, batch 64 x 300 steps, cross-entropy on spike counts): layer-layout kernels, the "
                         "transposing (rows, time) Functions, and the convolution / pooling / linear layers alone")
    ap.add_argument("--setup-only", action="store_true",
                    help="instead of the benchmark, make the ranges of the chosen --placement, print how long that took "
                         "and give them back")
    ap.add_argument("--placement", default="striped",
                    choices=["striped", "all-striped", "sorted-striped", "regions", "one-region", "plain"],
                    help="striped (default): sinabs.exodus.hbm.enable() as a program would call it -- the workload's inputs "
                         "come from the ordinary allocator, everything the kernels write lies in the striped range, whose "
                         "64 MiB pages alternate between the three regions of this GPU's HBM (a kernel's writes are held back "
                         "by the region they go to; spread over all three they are not).  all-striped: every big tensor in "
                         "the striped range -- a layer behind other layers, or hbm.enable(everything=True).  sorted-striped: "
                         "as striped, the ranges made with sort=True (timed copies decide which memory belongs to which "
                         "region).  regions / one-region: sorted ranges of one region each -- one region per tensor, and the "
                         "control with every tensor in the first region.  plain: the ordinary allocator.  The default run "
                         "reports striped, all-striped and plain (roofline.frac_by_placement); the plain figures are "
                         "measured first, in a child process, before this process touches the GPU")
    ap.add_argument("--region-map", type=float, nargs="?", const=4.0, default=0.0, metavar="GIB",
                    help="instead of the benchmark, fill device memory with buffers of GIB (default 4) GiB in the order "
                         "the driver hands them out, copy every buffer into every other with a flat copy kernel and print "
                         "the matrix of rates as text plus one JSON line with the region boundaries found")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (rows shard across GPUs without exchange; "
                 "no multi-GPU figure is produced). Run with --gpus 1.")

    if args.shape:
        b_, t_, m_ = (int(v) for v in args.shape.split(","))
        w_ = WORKLOADS[args.workload]
        WORKLOADS[args.workload] = dict(w_, batch=b_, steps=t_, neurons=m_,
                                        name=w_["name"] + f" -- at shape ({b_},{t_},{m_})")

    plain_first = None
    global SURROGATE
    SURROGATE = args.surrogate
    special = (args.region_map or args.ceilings or args.conv_snn or args.shape or args.copy_probe or args.setup_only
               or args.one_value_gradient or args.surrogate != "single")
    full_run = args.placement == "striped" and args.others == "all" and not special
    common = ["--no-cpu-baseline", "--workload", args.workload, "--path", args.path, "--steps", str(args.steps),
              "--warmup", str(args.warmup)]
    if full_run:
        # the same measurements with the ordinary allocator, in a process of its own and before this one touches
        # the GPU, so that it sees what a program that allocates without further thought is handed
        plain_first = child_json(["--placement", "plain", "--others", "api"] + common)

    import torch
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    from sinabs.exodus import _hip as hip
    from sinabs.exodus._compat import activation as act

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.one_lane_per_neuron or args.split_any_size:
        hip.backwardTimeSplit(0 if args.one_lane_per_neuron else 2)
    if args.region_map:
        measure_region_map(args, torch, dev)
        return
    place = Placement(torch, dev)
    placement_note = None
    if args.placement != "plain":
        from sinabs.exodus import hbm
        try:
            if args.placement == "one-region":
                place = Placement(torch, dev, hbm.enable(gib_per_region=40.0, gib_striped=0.0, device=dev, sort=True),
                                  mode="one-region")
            elif args.placement == "regions":
                place = Placement(torch, dev, hbm.enable(gib_per_region=32.0, gib_striped=0.0, device=dev, sort=True),
                                  mode="regions")
            elif args.placement == "sorted-striped":
                place = Placement(torch, dev, hbm.enable(gib_striped=72.0, device=dev, sort=True), mode="striped")
            else:
                place = Placement(torch, dev, hbm.enable(gib_striped=72.0, device=dev), mode=args.placement)
        except RuntimeError as err:                     # device memory in use by something else: measure without
            placement_note = f"ranges unavailable ({err}); ordinary allocator used"
            print("[bench] " + placement_note, file=sys.stderr, flush=True)
    if args.setup_only:
        out = dict(place.describe())
        if placement_note:
            out["placement_note"] = placement_note
        if place.regions is not None:
            if args.placement != "striped" and args.placement != "all-striped" and not place.regions.sorted:
                out["placement_note"] = ("timed copies found no three regions in the memory this process was handed (it comes "
                                         "mixed once other processes have used striped ranges): after retries with finer pieces "
                                         "the striped range was made unsorted, as sort=False makes it")
            out["gave_memory_back"] = hbm.disable()
        print(json.dumps(out))
        return
    if args.ceilings:
        print(json.dumps(measure_ceilings(args, torch, hip, dev, place)))
        return
    if args.conv_snn:
        print(json.dumps(dict(measure_conv_snn(args, torch, dev), **place.describe())))
        return
    if args.one_value_gradient and args.path != "layer":
        sys.exit("bench.py: --one-value-gradient goes with --path layer")
    if args.path == "layer":
        wl = build_layer_workload(args.workload, torch, hip, act, dev, place, one_value=args.one_value_gradient)
    else:
        wl = build_workload(args.workload, torch, hip, act, dev, place)
    fwd, bwd, N, T = wl["fwd"], wl["bwd"], wl["N"], wl["T"]

    if args.copy_probe:
        src = torch.ones(1 << 28, device=dev)          # 2^28 floats = 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        torch.neg(src, out=dst)                        # a plain elementwise kernel: 1 GiB in, 1 GiB out
        torch.cuda.synchronize()
        del src, dst

    m = measure(wl, args.steps, args.warmup, torch)
    ms_step, fwd_ms, bwd_ms = m["ms_per_step"], m["fwd_ms"], m["bwd_ms"]
    bf, bb = wl.get("bytes", WORKLOADS[args.workload]["bytes"])
    roof = roofline(args.workload, wl, fwd_ms, bwd_ms, bf, bb, traffic_known=not (args.shape or args.one_value_gradient))
    # how far single launches of this run lie apart (between processes the figures move by another 1-2 %, with where the
    # allocator put the tensors)
    dominant_is_bwd = bwd_ms >= fwd_ms
    roof["kernel_ms_min_max"] = m["bwd_ms_min_max"] if dominant_is_bwd else m["fwd_ms_min_max"]
    roof["other_kernel"]["kernel_ms_min_max"] = m["fwd_ms_min_max"] if dominant_is_bwd else m["bwd_ms_min_max"]
    # the same durations priced with the bytes of a kernel pair that stores and re-reads the states (the
    # figure the workload description quotes); "frac" uses what this design has to move, which is less
    # because the backward pass recomputes the states
    roof["priced_at_stored_state_bytes"] = {
        "bytes_per_neuron_timestep": sum(WORKLOADS[args.workload]["bytes"]),
        "fwd_bwd_combined_frac": N * T * sum(WORKLOADS[args.workload]["bytes"])
        / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS}

    result = {
        "metric": "neuron-timesteps/sec fwd+bwd (LIF, fp32) + % of HBM peak, 1 MI355X",
        "value": N * T / (ms_step * 1e-3),
        "unit": "neuron-timesteps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": WORKLOADS[args.workload]["name"], "path": args.path, "rows": N, "time_steps": T,
                   "algorithmic_bytes_per_neuron_timestep": bf + bb, **place.describe()},
        "roofline": roof,
    }
    if placement_note:
        result["config"]["placement_note"] = placement_note
    if args.surrogate != "single":
        result["config"]["surrogate"] = args.surrogate + " (a measurement aid: the configuration names SingleExponential)"
    if plain_first is not None:
        # the ordinary allocator's figures beside the headline: what the same kernels reach without hbm.enable()
        pr = plain_first.get("roofline", {})
        result["value_ordinary_allocator"] = plain_first.get("value")
        roof["frac_ordinary_allocator"] = pr.get("frac")
        roof["frac_by_placement"] = {
            "hbm.enable(): outputs striped over the three regions of HBM (this run's figures; the >= 70 % claim rests on it)":
                {"frac": roof["frac"], "fwd_bwd_combined_frac": roof["fwd_bwd_combined_frac"]},
            "ordinary allocator, first allocations of a process (measured before this one touched the GPU)":
                ({"frac": pr.get("frac"), "fwd_bwd_combined_frac": pr.get("fwd_bwd_combined_frac"),
                  "kernel_ms": pr.get("kernel_ms"), "other_kernel_ms": pr.get("other_kernel", {}).get("kernel_ms")}
                 if pr else plain_first)}
    del wl, fwd, bwd
    result["others"] = []
    if args.others == "all" and not args.shape:
        # the other configurations and the (rows, time) kernels behind the autograd Functions, a few
        # steps each: same measurement and placement, reported beside the headline workload
        for key, path in OTHERS:
            if (key, path) == (args.workload, args.path):
                continue
            other = (build_layer_workload if path == "layer" else build_workload)(key, torch, hip, act, dev, place)
            mo = measure(other, max(3, args.steps // 2), max(2, args.warmup // 2), torch)
            obf, obb = other.get("bytes", WORKLOADS[key]["bytes"])
            result["others"].append({
                "workload": WORKLOADS[key]["name"], "path": path, "rows": other["N"], "time_steps": other["T"],
                "steps": mo["steps"], "ms_per_step": mo["ms_per_step"],
                "value": other["N"] * other["T"] / (mo["ms_per_step"] * 1e-3), "unit": "neuron-timesteps/s",
                "algorithmic_bytes_per_neuron_timestep": obf + obb,
                "roofline": roofline(key, other, mo["fwd_ms"], mo["bwd_ms"], obf, obb)})
            del other
        # the headline workload with one number as the gradient of every spike (a sum as the loss)
        other = build_layer_workload(args.workload, torch, hip, act, dev, place, one_value=True)
        mo = measure(other, max(3, args.steps // 2), max(2, args.warmup // 2), torch)
        result["others"].append({
            "workload": WORKLOADS[args.workload]["name"] + " -- one value as the gradient of every output element",
            "path": "layer", "rows": other["N"], "time_steps": other["T"], "steps": mo["steps"],
            "ms_per_step": mo["ms_per_step"], "value": other["N"] * other["T"] / (mo["ms_per_step"] * 1e-3),
            "unit": "neuron-timesteps/s", "algorithmic_bytes_per_neuron_timestep": sum(other["bytes"]),
            "roofline": roofline(args.workload, other, mo["fwd_ms"], mo["bwd_ms"], *other["bytes"], traffic_known=False)})
        del other
    if args.others in ("all", "api") and not args.shape:
        # every configuration through the public layer API, with the ordinary allocator's figures (from the child
        # run) beside those of this process's placement
        plain_api = {(e.get("workload"), e.get("loss")): e for e in (plain_first or {}).get("others", [])
                     if str(e.get("path", "")).startswith("public layer API") and "loss" in e}
        steps_api, warm_api = max(3, args.steps // 2), max(2, args.warmup // 2)
        for key, loss in API_RUNS:
            e = measure_layer_api(key, loss, torch, dev, steps_api, warm_api, place_all=place.mode == "all-striped")
            e.update(place.describe())
            e.pop("placement_measured", None)
            twin = plain_api.get((e["workload"], e["loss"]))
            if twin:
                e["ordinary_allocator"] = {k: twin[k] for k in ("ms_per_step", "fwd_ms", "loss_ms", "bwd_ms", "value",
                                                                 "fwd_bwd_combined_frac")}
            result["others"].append(e)
    if args.others == "all" and not args.shape:
        small = measure_small_layer(torch, dev, args.steps, args.warmup)
        result["others"].append(small)
        conv = measure_conv_snn(argparse.Namespace(steps=max(3, args.steps // 4), warmup=2), torch, dev)
        result["others"].append(conv)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, torch)
    if full_run:
        # every tensor in the striped range, and the set-up time of ranges sorted by timed copies, each in a process
        # of its own once this one has given its memory back
        place = None
        import gc
        gc.collect()
        if not hbm.disable():
            print("[bench] the ranges could not be given back (tensors alive)", file=sys.stderr, flush=True)
        torch.cuda.empty_cache()
        torch.cuda.synchronize()
        allst = child_json(["--placement", "all-striped", "--others", "none"] + common)
        ar = allst.get("roofline")
        roof["frac_by_placement"]["every tensor striped over the three regions (measured last, in a process of its own)"] = (
            {"frac": ar["frac"], "fwd_bwd_combined_frac": ar["fwd_bwd_combined_frac"], "kernel_ms": ar["kernel_ms"],
             "other_kernel_ms": ar["other_kernel"]["kernel_ms"]} if ar else allst)
        # (last of all: by now the memory has been through the 64 MiB pages of two sets of ranges, and the sorting has
        # to cope with what it finds)
        result["placement_setup"] = {
            "hbm.enable() (default: sort=False), second process on the machine":
                {k: v for k, v in result["config"].items() if k.startswith("placement_setup")},
            "hbm.enable(sort=True), fourth process on the machine":
                child_json(["--placement", "sorted-striped", "--setup-only"])}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
