"""Regression pins: the committed vectors of tests/golden/function_cases.json against the CPU oracle
(CPU test) and against the HIP kernels through the autograd Functions (GPU test)."""
import json
import os

import pytest
import torch

from _util import assert_close


def unpack(d):
    if d is None:
        return None
    return torch.tensor([float.fromhex(h) for h in d["hex"]], dtype=torch.float32).reshape(d["shape"]).contiguous()


@pytest.fixture(scope="module")
def cases(golden_dir):
    with open(os.path.join(golden_dir, "function_cases.json")) as f:
        return json.load(f)["cases"]


def surrogate(mod, name):
    return {"single": mod.SingleExponential(), "periodic": mod.PeriodicExponential(), "heaviside": mod.Heaviside(0.6)}[name]


def test_oracle_reproduces_golden_vectors(cases):
    from oracle import exodus_ref as ref
    assert len(cases) >= 8
    for case in cases:
        i = {k: unpack(v) for k, v in case["inputs"].items()}
        o = {k: unpack(v) for k, v in case["outputs"].items()}
        if case["kind"] == "integrate_and_fire":
            s, v = ref.integrate_and_fire_forward(i["x"], i["alpha"], i["v0"], i["theta"], i["c"], i["lo"], case["cap"])
            assert torch.equal(s, o["spikes"]) and torch.equal(v, o["v_mem"]), case["name"]
            gi, ga, ginit = ref.integrate_and_fire_backward(i["go"], i["gv"], v, s, i["v0"], i["alpha"], i["c"], i["theta"],
                                                            i["lo"], surrogate(ref, case["surrogate"]), True,
                                                            gate_initial=True)
            assert torch.equal(gi, o["grad_input"]) and torch.equal(ga, o["grad_alpha"]) and torch.equal(ginit, o["grad_init"])
        else:
            out = ref.leaky_forward(i["x"], i["v0"], i["alpha"])
            assert torch.equal(out, o["out"]), case["name"]
            gi, ga, ginit = ref.leaky_integrator_backward(i["go"], out, i["v0"], i["alpha"], True)
            assert torch.equal(gi, o["grad_input"]) and torch.equal(ga, o["grad_alpha"]) and torch.equal(ginit, o["grad_init"])


@pytest.mark.gpu
def test_functions_match_golden_vectors(cases):
    from sinabs.exodus._compat import activation as act
    from sinabs.exodus.leaky import LeakyIntegrator
    from sinabs.exodus.spike import IntegrateAndFire
    for case in cases:
        i = {k: (None if v is None else unpack(v).cuda()) for k, v in case["inputs"].items()}
        o = {k: unpack(v) for k, v in case["outputs"].items()}
        x = i["x"].requires_grad_(True); alpha = i["alpha"].requires_grad_(True); v0 = i["v0"].requires_grad_(True)
        if case["kind"] == "integrate_and_fire":
            s, v = IntegrateAndFire.apply(x, alpha, v0, i["theta"], i["c"], i["lo"], surrogate(act, case["surrogate"]),
                                          case["cap"])
            assert torch.equal(s.cpu(), o["spikes"]) and torch.equal(v.detach().cpu(), o["v_mem"]), case["name"]
            ((s * i["go"]).sum() + (v * i["gv"]).sum()).backward()
        else:
            out = LeakyIntegrator.apply(x, alpha, v0)
            assert torch.equal(out.detach().cpu(), o["out"]), case["name"]
            (out * i["go"]).sum().backward()
        t = x.shape[1]
        assert_close(x.grad, o["grad_input"], case["name"] + " grad_input")
        assert_close(v0.grad, o["grad_init"], case["name"] + " grad_init")
        assert_close(alpha.grad, o["grad_alpha"], case["name"] + " grad_alpha", rtol=1e-4, atol=1e-5 * t ** 0.5)
