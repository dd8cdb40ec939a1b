"""Writes tests/golden/kat_vectors.npz: small known-answer vectors of the sync path.

Run in the CPU container from the repository root:  python tests/golden/make_kat_vectors.py
Inputs are seeded torch CPU randoms; expected outputs come from the pinned oracle
(oracle/oracle.py, itself checked by tests/test_oracle_pins.py). Nothing here runs or
imports reference code (the reference's Python needs an un-vendored submodule).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O   # noqa: E402

CASES = [
    # name, K, batches, n, dtype, std, opt
    ("k2_sgd", 2, (32, 32), 1200, "f32", 1e-3, dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                                                     groups=[dict(lr=0.1, weight_decay=1e-4)])),
    ("k4_adamw", 4, (48, 32, 32, 16), 1100, "f32", 5e-4, dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
                                                               groups=[dict(lr=5e-4, weight_decay=0.05)])),
    ("k3_sgd", 3, (4, 2, 2), 515, "f32", 1e-3, dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                                                      groups=[dict(lr=0.02, weight_decay=1e-4)])),
    ("k4_adam", 4, (128, 128, 64, 64), 1030, "f32", 1e-3, dict(kind="adam", betas=(0.9, 0.999), eps=1e-8,
                                                                groups=[dict(lr=2e-3, weight_decay=0.0)])),
    ("k8_bf16_adamw", 8, tuple(range(64, 0, -8)), 1100, "bf16", 2e-4,
     dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8, groups=[dict(lr=5e-4, weight_decay=0.05)])),
]


def main():
    out = {}
    for ci, (name, K, batches, n, dt, std, opt) in enumerate(CASES):
        gen = torch.Generator().manual_seed(1234 + 17 * ci)
        grads = [(torch.randn(n, generator=gen) * std) for _ in range(K)]
        if dt == "bf16":
            grads = [g.to(torch.bfloat16) for g in grads]
        if name == "k4_adam":                         # rows of exact zeros, as a sparse embedding gradient has
            for g in grads:
                g[256:768] = 0.0
        p = torch.randn(n, generator=gen) * 0.05
        s1, s2 = torch.zeros(n), torch.zeros(n)
        out[f"{name}/p0"] = p.numpy().copy()
        for k, g in enumerate(grads):
            out[f"{name}/g{k}"] = (g.view(torch.int16) if dt == "bf16" else g).numpy().copy()
        work = [g.clone() for g in grads]
        for step in (1, 2):
            agg, rows = O.sync_step(work, batches, [(0, n, ((0, 0),))], opt, p, s1, s2 if opt["kind"] != "sgd" else None,
                                    step=step, first_step=(step == 1), want_stats=True)
            out[f"{name}/agg{step}"] = agg.numpy().copy()
            out[f"{name}/stats{step}"] = rows[0].numpy().copy()
            if step == 2:
                out[f"{name}/p2"] = p.numpy().copy()
                out[f"{name}/s1_2"] = s1.numpy().copy()
                out[f"{name}/s2_2"] = s2.numpy().copy()
            if dt == "f32":
                work[0] = agg.clone()                 # in place: VSW 0's bucket now holds the aggregate
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
