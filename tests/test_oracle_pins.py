"""Pins the CPU oracle (oracle/oracle.py) before anything is compared with it.

The reference ships no tests or golden vectors for this path, so each oracle function is
checked against (a) an independent scalar C restatement, bit for bit, (b) scalar
numpy.float32 brute force on tiny inputs, (c) library routines (torch.optim.*,
torch.nn.functional.cosine_similarity, float64 dot), (d) closed forms and invariants
chosen so that a dropped term, a swapped operand or a wrong sign fails one of them.
"""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import c_oracle as OC


def _grads(K, n, seed, std=1e-3, dtype=torch.float32):
    out = []
    for k in range(K):
        g = torch.Generator().manual_seed(1234 + 17 * seed + k)
        out.append((torch.randn(n, generator=g) * std).to(dtype))
    return out


def _bits(t):
    return t.contiguous().view(torch.int32)


BATCHES = {1: (32,), 2: (32, 32), 3: (4, 2, 2), 4: (48, 32, 32, 16), 5: (5, 4, 3, 2, 1),
           6: (7, 7, 5, 3, 2, 1), 7: (64, 56, 48, 40, 32, 24, 16), 8: tuple(range(64, 0, -8)),
           9: (9, 8, 7, 6, 5, 4, 3, 2, 1), 12: (32, 16, 8) * 4, 13: tuple(range(1, 14)),
           16: tuple(range(64, 0, -4))}


# ------------------------------------------------------------------------------ weights
def test_batch_weights_are_double_quotients_rounded_once():
    w, hid, hw = O.batch_weights((48, 32, 32, 16))
    assert w == [float(np.float32(48 / 128)), 0.25, 0.25, 0.125]
    assert hid == [0, 1, 0, 1]
    assert hw == [float(np.float32(48 / 80)), float(np.float32(32 / 48)), float(np.float32(32 / 80)),
                  float(np.float32(16 / 48))]
    w3, _, _ = O.batch_weights((4, 2, 2))
    assert w3 == [0.5, 0.25, 0.25]


# ---------------------------------------------------------------------------- aggregate
@pytest.mark.parametrize("K", list(range(1, 9)) + [9, 12, 13, 16])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_aggregate_matches_c_restatement_bitwise(K, dtype):
    g = _grads(K, 4099, K, dtype=dtype)
    w, _, _ = O.batch_weights(BATCHES[K])
    a = O.aggregate(g, BATCHES[K])
    b = OC.aggregate(g, w)
    assert torch.equal(_bits(a), _bits(b))


def test_aggregate_brute_force_numpy_scalar():
    K, n = 4, 37
    g = _grads(K, n, 3)
    w, _, _ = O.batch_weights(BATCHES[K])
    got = O.aggregate(g, BATCHES[K]).numpy()
    for i in range(n):
        acc = np.float32(g[0][i].item()) * np.float32(w[0])
        for k in range(1, K):
            acc = np.float32(acc + np.float32(np.float32(g[k][i].item()) * np.float32(w[k])))
        assert acc.tobytes() == got[i].tobytes()


def test_aggregate_k1_is_identity():
    g = _grads(1, 1000, 5)
    assert torch.equal(_bits(O.aggregate(g, (32,))), _bits(g[0]))


@pytest.mark.parametrize("K", [2, 4, 8, 16])
def test_aggregate_equal_batches_power_of_two_is_sum_then_divide(K):
    # the reference's own pattern: sum over workers, then one division by the count
    # (similarity_allreduce.py:32); exact for power-of-two counts
    g = _grads(K, 5000, 7)
    acc = g[0].clone()
    for k in range(1, K):
        acc = acc + g[k]
    ref = acc / K
    assert torch.equal(_bits(O.aggregate(g, (16,) * K)), _bits(ref))


def test_aggregate_equal_batches_k3_within_k_ulp_of_sum_then_divide():
    g = _grads(3, 5000, 9)
    ref = ((g[0] + g[1]) + g[2]) / 3
    got = O.aggregate(g, (8, 8, 8))
    # rounding errors scale with the operands, not with the (possibly cancelling) sum
    ulp = (g[0].abs() + g[1].abs() + g[2].abs()) / 3 * 2.0 ** -23
    assert torch.all(torch.abs(got - ref) <= 3 * ulp)


def test_aggregate_keeps_exact_zero_rows_positive_zero():
    g = _grads(4, 4096, 11)
    for t in g:
        t[1000:3000] = 0.0
    out = O.aggregate(g, BATCHES[4])
    assert torch.all(_bits(out[1000:3000]) == 0)


def test_aggregate_order_matters_only_within_rounding():
    g = _grads(4, 4096, 13)
    a = O.aggregate(g, (48, 32, 32, 16))
    b = O.aggregate(list(reversed(g)), (16, 32, 32, 48))
    assert not torch.equal(_bits(a), _bits(b))          # documented: order changes bits
    ulp = sum(t.abs() for t in g) / 4 * 2.0 ** -23
    assert torch.all(torch.abs(a - b) <= 4 * ulp)


def test_bf16_widening_is_exact():
    g = _grads(2, 1024, 15, dtype=torch.bfloat16)
    wide = [t.float() for t in g]
    assert torch.equal(_bits(O.aggregate(g, (3, 1))), _bits(O.aggregate(wide, (3, 1))))


# --------------------------------------------------------------------------- statistics
@pytest.mark.parametrize("K", [1, 2, 3, 4, 8, 9, 13, 16])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stats_match_c_restatement(K, dtype):
    g = _grads(K, 10007, 20 + K, dtype=dtype)
    w, hid, hw = O.batch_weights(BATCHES[K])
    a = O.stats(g, BATCHES[K])
    b = OC.stats(g, w, hid, hw)
    assert torch.allclose(a, b, rtol=1e-12, atol=1e-30)


def test_stats_against_library_cosine_float64():
    K = 4
    g = _grads(K, 20000, 31, std=5e-4)
    row = O.stats(g, BATCHES[K])
    ga, gb = O.half_aggregates(g, BATCHES[K])
    lib = torch.nn.functional.cosine_similarity(ga.double(), gb.double(), dim=0).item()
    assert O.cosine(row[O.DOT_AB].item(), row[O.NORM_A].item(), row[O.NORM_B].item()) == pytest.approx(lib, rel=1e-12)
    # the halves are the batch-weighted means of the even / odd workers
    ea = (48 * g[0].double() + 32 * g[2].double()) / 80
    eb = (32 * g[1].double() + 16 * g[3].double()) / 48
    assert torch.allclose(ga.double(), ea, rtol=1e-6, atol=5e-10)
    assert torch.allclose(gb.double(), eb, rtol=1e-6, atol=5e-10)


def test_stats_textbook_identities():
    g0 = _grads(1, 5000, 33)[0]
    same = O.stats([g0, g0.clone()], (8, 8))
    assert O.cosine_from_rows(same) == pytest.approx(1.0, abs=1e-12)
    opp = O.stats([g0, -g0], (8, 8))
    assert O.cosine_from_rows(opp) == pytest.approx(-1.0, abs=1e-12)
    assert opp[O.NORM_AGG].item() == 0.0                      # g - g cancels exactly
    e0, e1 = torch.zeros(64), torch.zeros(64)
    e0[3], e1[40] = 2.0, -5.0
    orth = O.stats([e0, e1], (1, 1))
    assert orth[O.DOT_AB].item() == 0.0 and O.cosine_from_rows(orth) == 0.0
    assert orth[O.NORM_VSW0].item() == 4.0 and orth[O.NORM_VSW0 + 1].item() == 25.0
    # scale invariance of the cosine (power-of-two scale keeps every rounding identical)
    g = _grads(2, 5000, 35)
    c1 = O.cosine_from_rows(O.stats(g, (3, 5)))
    c2 = O.cosine_from_rows(O.stats([g[0] * 4, g[1] * 4], (3, 5)))
    assert c1 == pytest.approx(c2, rel=1e-14)
    # zero gradient: clamp by eps^2 gives 0, not NaN
    z = torch.zeros(100)
    assert O.cosine_from_rows(O.stats([z, z], (1, 1))) == 0.0


def test_stats_sum_over_buckets_is_whole_model_value():
    K = 4
    g = _grads(K, 9000, 37)
    cuts = [0, 1000, 1003, 6000, 9000]
    rows = torch.stack([O.stats([t[a:b] for t in g], BATCHES[K]) for a, b in zip(cuts, cuts[1:])])
    whole = O.stats(g, BATCHES[K])
    assert torch.allclose(rows.sum(0), whole, rtol=1e-12)
    ga, gb = O.half_aggregates(g, BATCHES[K])
    lib = torch.nn.functional.cosine_similarity(ga.double(), gb.double(), dim=0).item()
    assert O.cosine_from_rows(rows) == pytest.approx(lib, rel=1e-12)


def test_gram_symmetric_diag_is_worker_norms_and_matches_c():
    K = 5
    g = _grads(K, 3001, 39)
    G = O.gram(g)
    assert torch.allclose(G, G.t())
    row = O.stats(g, BATCHES[K])
    assert torch.allclose(torch.diagonal(G), row[O.NORM_VSW0:O.NORM_VSW0 + K], rtol=1e-12)
    assert torch.allclose(G, OC.gram(g), rtol=1e-12, atol=1e-30)
    assert G[1, 3].item() == pytest.approx(torch.dot(g[1].double(), g[3].double()).item(), rel=1e-12)


# ---------------------------------------------------------------------------------- SGD
SGD_CASES = [
    dict(lr=0.1, weight_decay=1e-4, momentum=0.9, dampening=0.0, nesterov=False),
    dict(lr=0.02, weight_decay=0.0, momentum=0.9, dampening=0.0, nesterov=False),
    dict(lr=0.05, weight_decay=5e-4, momentum=0.8, dampening=0.0, nesterov=True),
    dict(lr=0.05, weight_decay=1e-3, momentum=0.7, dampening=0.3, nesterov=False),
    dict(lr=0.3, weight_decay=1e-2, momentum=0.0, dampening=0.0, nesterov=False),
]


def _state(n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, generator=g) * 0.05


@pytest.mark.parametrize("hp", SGD_CASES)
def test_sgd_matches_c_bitwise_and_torch_optim(hp):
    n, steps = 3001, 4
    p_o, p_c = _state(n, 1), _state(n, 1)
    p_t = torch.nn.Parameter(_state(n, 1))
    buf_o, buf_c = torch.zeros(n), torch.zeros(n)
    opt = torch.optim.SGD([p_t], foreach=False, **hp)
    for s in range(steps):
        g = _grads(1, n, 50 + s)[0]
        O.sgd_step(p_o, g, buf_o, first_step=(s == 0), **hp)
        OC.sgd_step(p_c, g, buf_c, first_step=(s == 0), **hp)
        p_t.grad = g.clone()
        opt.step()
        assert torch.equal(_bits(p_o), _bits(p_c))
        assert torch.equal(_bits(buf_o), _bits(buf_c))
    assert torch.allclose(p_o, p_t.detach(), rtol=1e-6, atol=1e-9)
    if hp["momentum"]:
        assert torch.allclose(buf_o, opt.state[p_t]["momentum_buffer"], rtol=1e-6, atol=2e-9)


def test_sgd_first_step_closed_form():
    n = 1000
    p0, g = _state(n, 2), _grads(1, n, 60)[0]
    p, buf = p0.clone(), torch.zeros(n)
    O.sgd_step(p, g, buf, lr=0.1, weight_decay=1e-4, momentum=0.9, first_step=True)
    d = g.double() + 1e-4 * p0.double()
    assert torch.allclose(p.double(), p0.double() - 0.1 * d, rtol=1e-6, atol=1e-10)
    assert torch.allclose(buf.double(), d, rtol=1e-6, atol=1e-12)         # buf = d, not (1-damp)*d


# --------------------------------------------------------------------------------- Adam
ADAM_CASES = [
    dict(lr=5e-4, weight_decay=0.05, betas=(0.9, 0.999), eps=1e-8, adamw=True),
    dict(lr=5e-4, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, adamw=True),
    dict(lr=2e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, adamw=False),
    dict(lr=1e-3, weight_decay=1e-2, betas=(0.8, 0.99), eps=1e-6, adamw=False),
]


@pytest.mark.parametrize("hp", ADAM_CASES)
def test_adam_matches_c_bitwise_and_torch_optim(hp):
    n, steps = 3001, 5
    p_o, p_c = _state(n, 3), _state(n, 3)
    p_t = torch.nn.Parameter(_state(n, 3))
    m_o, v_o, m_c, v_c = torch.zeros(n), torch.zeros(n), torch.zeros(n), torch.zeros(n)
    cls = torch.optim.AdamW if hp["adamw"] else torch.optim.Adam
    opt = cls([p_t], lr=hp["lr"], weight_decay=hp["weight_decay"], betas=hp["betas"], eps=hp["eps"], foreach=False)
    for s in range(1, steps + 1):
        g = _grads(1, n, 70 + s, std=5e-4)[0]
        O.adam_step(p_o, g, m_o, v_o, step=s, **hp)
        OC.adam_step(p_c, g, m_c, v_c, step=s, **hp)
        p_t.grad = g.clone()
        opt.step()
        for a, b in ((p_o, p_c), (m_o, m_c), (v_o, v_c)):
            assert torch.equal(_bits(a), _bits(b))
    assert torch.allclose(p_o, p_t.detach(), rtol=1e-6, atol=1e-9)
    assert torch.allclose(m_o, opt.state[p_t]["exp_avg"], rtol=1e-6, atol=2e-10)
    assert torch.allclose(v_o, opt.state[p_t]["exp_avg_sq"], rtol=1e-6, atol=1e-16)


def test_adam_first_step_closed_form_is_sign_step():
    n = 2000
    p0, g = _state(n, 4), _grads(1, n, 80)[0]
    p, m, v = p0.clone(), torch.zeros(n), torch.zeros(n)
    O.adam_step(p, g, m, v, lr=2e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, step=1, adamw=False)
    expect = p0.double() - 2e-3 * g.double() / (g.double().abs() + 1e-8)
    assert torch.allclose(p.double(), expect, rtol=2e-6, atol=1e-9)
    assert torch.allclose(m.double(), 0.1 * g.double(), rtol=1e-6)
    assert torch.allclose(v.double(), 0.001 * g.double() ** 2, rtol=1e-5)


def test_adam_zero_gradient_decays_moments_geometrically():
    n = 512
    p, m, v = _state(n, 5), _state(n, 6).abs(), _state(n, 7).abs()
    m0, v0 = m.clone(), v.clone()
    z = torch.zeros(n)
    for s in range(1, 4):
        O.adam_step(p, z, m, v, lr=1e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, step=s, adamw=False)
    assert torch.allclose(m.double(), m0.double() * 0.9 ** 3, rtol=1e-6)
    assert torch.allclose(v.double(), v0.double() * 0.999 ** 3, rtol=1e-6)


def test_adamw_decay_is_decoupled():
    n = 256
    p0 = _state(n, 8)
    z = torch.zeros(n)
    p, m, v = p0.clone(), torch.zeros(n), torch.zeros(n)
    O.adam_step(p, z, m, v, lr=5e-4, weight_decay=0.05, betas=(0.9, 0.999), eps=1e-8, step=1, adamw=True)
    assert torch.allclose(p.double(), p0.double() * (1 - 5e-4 * 0.05), rtol=1e-6)
    assert torch.count_nonzero(m) == 0 and torch.count_nonzero(v) == 0     # decay never enters the moments


@pytest.mark.parametrize("hp", ADAM_CASES)
def test_amsgrad_matches_c_bitwise_and_torch_optim(hp):
    """amsgrad as ShardGNMTAdam.step threads it into F.adam (examples/gnmt/seq2seq/train/shard_optimizer.py:58-66,
    79-90): both restatements bit for bit, torch.optim.Adam / AdamW(amsgrad=True) as the library routine. The
    gradients shrink after the second step, so the second moment falls below its maximum and a denominator
    taken from the moment instead of the maximum would show."""
    n, steps = 3001, 6
    p_o, p_c, p_plain = _state(n, 3), _state(n, 3), _state(n, 3)
    p_t = torch.nn.Parameter(_state(n, 3))
    m_o, v_o, x_o, m_c, v_c, x_c = (torch.zeros(n) for _ in range(6))
    m_p, v_p = torch.zeros(n), torch.zeros(n)
    cls = torch.optim.AdamW if hp["adamw"] else torch.optim.Adam
    opt = cls([p_t], lr=hp["lr"], weight_decay=hp["weight_decay"], betas=hp["betas"], eps=hp["eps"], foreach=False,
              amsgrad=True)
    history = []
    for s in range(1, steps + 1):
        g = _grads(1, n, 170 + s, std=5e-3 if s <= 2 else 2e-4)[0]
        O.adam_step(p_o, g, m_o, v_o, step=s, vmax=x_o, **hp)
        OC.adam_step(p_c, g, m_c, v_c, step=s, vmax=x_c, **hp)
        O.adam_step(p_plain, g, m_p, v_p, step=s, **hp)
        history.append(v_o.clone())
        p_t.grad = g.clone()
        opt.step()
        for a, b in ((p_o, p_c), (m_o, m_c), (v_o, v_c), (x_o, x_c)):
            assert torch.equal(_bits(a), _bits(b))
        assert torch.equal(_bits(x_o), _bits(torch.stack(history).max(dim=0).values))      # the running maximum, exactly
    assert torch.allclose(p_o, p_t.detach(), rtol=1e-6, atol=1e-9)
    assert torch.allclose(m_o, opt.state[p_t]["exp_avg"], rtol=1e-6, atol=2e-10)
    assert torch.allclose(v_o, opt.state[p_t]["exp_avg_sq"], rtol=1e-6, atol=1e-16)
    assert torch.allclose(x_o, opt.state[p_t]["max_exp_avg_sq"], rtol=1e-6, atol=1e-16)
    if hp["adamw"] or hp["weight_decay"] == 0:            # (L2 decay feeds the weights back into the moments)
        assert torch.equal(_bits(v_o), _bits(v_p)) and torch.equal(_bits(m_o), _bits(m_p))     # the moments are Adam's own
    assert (x_o > v_o).float().mean() > 0.5                 # the maximum is what the last steps mostly divided by ...
    assert not torch.allclose(p_o, p_plain, rtol=1e-6, atol=1e-9)                          # ... and it shows in the weights


def test_amsgrad_maximum_propagates_nan_like_torch_maximum():
    n = 8
    g = torch.full((n,), 1e-3)
    g[3] = float("nan")
    outs = []
    for mod in (O, OC):
        p, m, v, x = torch.ones(n), torch.zeros(n), torch.zeros(n), torch.full((n,), 1e-3)
        mod.adam_step(p, g, m, v, lr=1e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, step=1, adamw=False, vmax=x)
        assert torch.isnan(x[3]) and torch.isnan(p[3]) and not torch.isnan(x[[0, 1, 2, 4, 5, 6, 7]]).any()
        assert torch.equal(x[:3], torch.full((3,), 1e-3))    # the old maximum stands where the moment is below it
        outs.append((p, x))
    assert torch.equal(_bits(outs[0][0]), _bits(outs[1][0])) and torch.equal(_bits(outs[0][1]), _bits(outs[1][1]))


# --------------------------------------------------------------------- composite step
def test_sync_step_composes_pieces_per_span_and_group():
    K, n = 3, 5000
    g = _grads(K, n, 90)
    spans = [(0, 1200, ((0, 1), (700, 0))), (1200, 3800, ((0, 0), (100, 1), (3000, 0)))]
    opt = dict(kind="sgd", momentum=0.9, groups=[dict(lr=0.1, weight_decay=0.0), dict(lr=0.1, weight_decay=1e-4)])
    p, buf = _state(n, 9), torch.zeros(n)
    p0 = p.clone()
    agg, rows = O.sync_step(g, BATCHES[K], spans, opt, p, buf, None, step=1, first_step=True, want_stats=True)
    assert torch.equal(_bits(agg), _bits(O.aggregate(g, BATCHES[K])))
    assert torch.allclose(rows.sum(0), O.stats(g, BATCHES[K]), rtol=1e-12)
    # group 0 stretch: no weight decay; group 1 stretch: weight decay 1e-4
    nd = slice(700, 1200)
    assert torch.allclose(p[nd].double(), p0[nd].double() - 0.1 * agg[nd].double(), rtol=1e-6, atol=1e-10)
    wd = slice(0, 700)
    assert torch.allclose(p[wd].double(), p0[wd].double() - 0.1 * (agg[wd].double() + 1e-4 * p0[wd].double()),
                          rtol=1e-6, atol=1e-10)


# ----------------------------------------------------------------------------- clipping
@pytest.mark.parametrize("max_norm", [0.01, 5.0])
def test_clip_matches_torch_clip_grad_norm(max_norm):
    shapes = [(300,), (17, 31), (1000,)]
    gen = torch.Generator().manual_seed(5)
    params = [torch.nn.Parameter(torch.zeros(s)) for s in shapes]
    for p in params:
        p.grad = torch.randn(p.shape, generator=gen) * 1e-2
    flat = torch.cat([p.grad.reshape(-1) for p in params]).clone()
    total = torch.nn.utils.clip_grad_norm_(params, max_norm)
    got, c = O.clip(flat, max_norm)
    want = torch.cat([p.grad.reshape(-1) for p in params])
    assert float(total) == pytest.approx(math.sqrt(float(torch.dot(flat.double(), flat.double()))), rel=1e-6)
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-12)
    if max_norm == 5.0:
        assert c > 1.0 and torch.equal(got, flat)              # above the norm: untouched, bit for bit
    else:
        assert c < 1.0 and float(torch.linalg.vector_norm(got.double())) == pytest.approx(max_norm, rel=1e-4)


def test_accumulated_micro_batches_count_as_decoupled_workers():
    """With A micro-batches summed into every bucket the divisor grows by A (the reference's
    global batch = local batch x decoupled workers, jabas/train/trainer.py:594-599)."""
    w, hid, hw = O.batch_weights((4, 2, 2), accumulations=2)
    assert w == [0.25, 0.125, 0.125] and hid == [0, 1, 0]
    assert hw == [float(np.float32(4 / 12)), 0.5, float(np.float32(2 / 12))]
    from jabas_amd import sync
    w2, hid2, hw2 = sync.batch_weights((4, 2, 2), accumulations=2)
    assert [float(x) for x in w2] == w and [float(x) for x in hw2] == hw
    with pytest.raises(ValueError):
        sync.batch_weights((4, 2), accumulations=0)
    # equal batches, power-of-two count: accumulating twice equals one worker set of twice the size
    g = _grads(2, 1000, 77)
    summed = [torch.add(g[0], g[1]), torch.add(g[1], g[0])]                 # two micro-batches per worker
    w4, _, _ = O.batch_weights((8, 8), accumulations=2)
    got = torch.add(torch.mul(summed[0], w4[0]), torch.mul(summed[1], w4[1]))
    want = O.aggregate([g[0], g[1], g[1], g[0]], (8, 8, 8, 8))
    assert torch.allclose(got, want, rtol=0, atol=float(torch.finfo(torch.float32).eps) * float(want.abs().max()) * 4)
