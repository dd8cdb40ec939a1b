"""Known-answer vectors (tests/golden/kat_vectors.npz): the oracle must still produce
them (CPU), and the HIP path must produce them through the C ABI (GPU). Aggregate
bit-exact; statistics 1e-6 relative (1e-2 for bf16 inputs); weights and state 1e-6."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.golden.make_kat_vectors import CASES

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat_vectors.npz")


def _load(name, K, dt):
    z = np.load(PATH, allow_pickle=False)
    grads = []
    for k in range(K):
        g = torch.from_numpy(z[f"{name}/g{k}"].copy())
        grads.append(g.view(torch.bfloat16) if dt == "bf16" else g)
    return z, grads


def _close(a, b, rtol, atol):
    a, b = torch.as_tensor(a).double(), torch.as_tensor(b).double()
    return bool(((a - b).abs() <= rtol * b.abs() + atol).all())


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_oracle_reproduces_the_vectors(case):
    name, K, batches, n, dt, std, opt = case
    z, grads = _load(name, K, dt)
    p = torch.from_numpy(z[f"{name}/p0"].copy())
    s1, s2 = torch.zeros(n), torch.zeros(n)
    work = [g.clone() for g in grads]
    for step in (1, 2):
        agg, rows = O.sync_step(work, batches, [(0, n, ((0, 0),))], opt, p, s1, s2 if opt["kind"] != "sgd" else None,
                                step=step, first_step=(step == 1), want_stats=True)
        assert np.array_equal(agg.numpy().view(np.int32), z[f"{name}/agg{step}"].view(np.int32))
        want = torch.as_tensor(z[f"{name}/stats{step}"])           # the fixture rows hold 4 + 8 slots
        assert _close(rows[0][:want.numel()], want, 1e-12, 0.0)
        assert torch.count_nonzero(rows[0][want.numel():]) == 0
        if dt == "f32":
            work[0] = agg.clone()
    assert np.array_equal(p.numpy().view(np.int32), z[f"{name}/p2"].view(np.int32))
    assert np.array_equal(s1.numpy().view(np.int32), z[f"{name}/s1_2"].view(np.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_hip_path_reproduces_the_vectors(gpu, case):
    from jabas_amd import sync
    name, K, batches, n, dt, std, opt = case
    z, grads = _load(name, K, dt)
    gdt = torch.bfloat16 if dt == "bf16" else torch.float32
    dg = [g.to(gpu) for g in grads]
    agg_d = dg[0] if dt == "f32" else torch.zeros(n, device=gpu)
    p = torch.from_numpy(z[f"{name}/p0"].copy()).to(gpu)
    s1, s2 = torch.zeros(n, device=gpu), torch.zeros(n, device=gpu)
    adam = opt["kind"] != "sgd"
    span = sync.SpanSpec(dg, agg_out=agg_d, param=p, state1=s1, state2=s2 if adam else None, bounds=((0, 0),))
    for step in (1, 2):
        args = sync.make_step_args(batches, gdt, stats=True, opt=opt, step=step, first_step=(step == 1))
        row = sync.sync_bucket(span, args)
        torch.cuda.synchronize()
        assert np.array_equal(agg_d.cpu().numpy().view(np.int32), z[f"{name}/agg{step}"].view(np.int32)), step
        rtol = 1e-2 if dt == "bf16" else 1e-6
        assert _close(row.cpu()[:4 + K], z[f"{name}/stats{step}"][:4 + K], rtol, 0.0)
    assert _close(p.cpu(), z[f"{name}/p2"], 1e-6, 1e-9)
    assert _close(s1.cpu(), z[f"{name}/s1_2"], 1e-6, 2e-9)
    if adam:
        assert _close(s2.cpu(), z[f"{name}/s2_2"], 1e-6, 1e-16)
