"""Writes tests/golden/function_cases.json: small seeded inputs with the outputs of the CPU oracle
(oracle/exodus_ref.py) for each Function and flag combination.

Run from the repository root after tests/test_oracle_pins.py passes:

    python tests/golden/make_function_cases.py

The vectors are a regression pin: they freeze what the pinned oracle computed when they were made,
so that later changes to the oracle or to the kernels are noticed.  Values are stored as hex floats
(exact fp32 bits)."""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import exodus_ref as ref  # noqa: E402


def hexlist(t):
    return [float(v).hex() for v in t.detach().flatten().tolist()]


def pack(t):
    return {"shape": list(t.shape), "hex": hexlist(t)}


def main():
    g = torch.Generator().manual_seed(20240)
    cases = []
    n, t = 6, 24
    for idx, (cap, use_lo, surr) in enumerate([(None, False, "single"), (1, True, "single"), (2, True, "periodic"),
                                               (None, True, "heaviside"), (3, False, "periodic")]):
        x = torch.randn(n, t, generator=g) * 0.7 + 0.25
        alpha = torch.rand(n, generator=g); v0 = torch.randn(n, generator=g) * 0.3
        th = 0.5 + torch.rand(n, generator=g); c = 0.3 + 0.5 * torch.rand(n, generator=g)
        lo = -0.2 - 0.3 * torch.rand(n, generator=g) if use_lo else None
        go = torch.randn(n, t, generator=g); gv = torch.randn(n, t, generator=g)
        fn = {"single": ref.SingleExponential(), "periodic": ref.PeriodicExponential(), "heaviside": ref.Heaviside(0.6)}[surr]
        s, v = ref.integrate_and_fire_forward(x, alpha, v0, th, c, lo, cap)
        gi, ga, ginit = ref.integrate_and_fire_backward(go, gv, v, s, v0, alpha, c, th, lo, fn, True, gate_initial=True)
        cases.append(dict(kind="integrate_and_fire", name=f"iaf_{idx}", cap=cap, surrogate=surr,
                          inputs=dict(x=pack(x), alpha=pack(alpha), v0=pack(v0), theta=pack(th), c=pack(c),
                                      lo=None if lo is None else pack(lo), go=pack(go), gv=pack(gv)),
                          outputs=dict(spikes=pack(s), v_mem=pack(v), grad_input=pack(gi), grad_alpha=pack(ga),
                                       grad_init=pack(ginit))))
    for idx in range(3):
        x = torch.randn(n, t, generator=g); alpha = torch.rand(n, generator=g); v0 = torch.randn(n, generator=g)
        go = torch.randn(n, t, generator=g)
        out = ref.leaky_forward(x, v0, alpha)
        gi, ga, ginit = ref.leaky_integrator_backward(go, out, v0, alpha, True)
        cases.append(dict(kind="leaky", name=f"leaky_{idx}",
                          inputs=dict(x=pack(x), alpha=pack(alpha), v0=pack(v0), go=pack(go)),
                          outputs=dict(out=pack(out), grad_input=pack(gi), grad_alpha=pack(ga), grad_init=pack(ginit))))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "function_cases.json")
    with open(path, "w") as f:
        json.dump(dict(made_by="tests/golden/make_function_cases.py", cases=cases), f)
    print(path, len(cases), "cases")


if __name__ == "__main__":
    main()
