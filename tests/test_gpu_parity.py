"""GPU parity: the HIP path, called through the C ABI (ctypes), against the CPU oracle on
the same seeded inputs. Bars (from the path's specification):
  aggregate            bit-exact (fp32 and bf16 inputs)
  statistics           1e-6 relative (fp32 inputs), 1e-2 relative (bf16 inputs)
  updated weights/state 1e-6 relative (plus an absolute floor of a few ulp of the operands,
                       because m and buf are sums that may cancel)
The optimizer checks additionally report how many elements are bit-identical.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

BATCHES = {1: (32,), 2: (32, 32), 3: (4, 2, 2), 4: (48, 32, 32, 16), 5: (5, 4, 3, 2, 1),
           6: (7, 7, 5, 3, 2, 1), 7: (64, 56, 48, 40, 32, 24, 16), 8: tuple(range(64, 0, -8)),
           9: (9, 8, 7, 6, 5, 4, 3, 2, 1), 10: (16,) * 10, 11: tuple(range(11, 0, -1)), 12: (32, 16, 8) * 4,
           13: tuple(range(1, 14)), 14: (3, 5) * 7, 15: tuple(range(30, 0, -2)), 16: tuple(range(64, 0, -4))}

SGD = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
           groups=[dict(lr=0.1, weight_decay=0.0), dict(lr=0.1, weight_decay=1e-4)])
ADAMW = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
             groups=[dict(lr=5e-4, weight_decay=0.0), dict(lr=5e-4, weight_decay=0.05)])
ADAM = dict(kind="adam", betas=(0.9, 0.999), eps=1e-8, groups=[dict(lr=2e-3, weight_decay=0.0),
                                                                dict(lr=2e-3, weight_decay=1e-2)])


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int32)


def _host_grads(K, n, seed, std=1e-3, dtype=torch.float32):
    out = []
    for k in range(K):
        g = torch.Generator().manual_seed(1234 + 17 * seed + k)
        out.append((torch.randn(n, generator=g) * std).to(dtype))
    return out


def _host_state(n, seed, scale=0.05):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, generator=g) * scale


def _dev(t, gpu, skew=0):
    """Device copy of t placed `skew` elements into a 256-byte aligned allocation."""
    buf = torch.zeros(t.numel() + 128, dtype=t.dtype, device=gpu)
    view = buf[skew:skew + t.numel()]
    view.copy_(t)
    return view


def _close(got, want, rtol, atol):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    err = (got - want).abs()
    ok = err <= rtol * want.abs() + atol
    return bool(ok.all()), float(err.max()) if err.numel() else 0.0


def _same_bits(a, b):
    a, b = _bits(a), _bits(b)
    return int((a == b).sum()), a.numel()


# ---------------------------------------------------------------------------- aggregate
@pytest.mark.parametrize("K", range(1, 17))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_aggregate_bit_exact(gpu, K, dtype):
    from jabas_amd import sync
    for n, skew in ((1, 0), (3, 1), (1023, 0), (1024, 2), (1025, 3), (4099, 0), (262144 + 77, 0), (1 << 20, 3),
                    (4099, 37), (70001, 63), (5, 61)):
        print(f"aggregate K={K} {dtype} n={n} skew={skew}", flush=True)
        hg = _host_grads(K, n, K + n % 7, dtype=dtype)
        dg = [_dev(t, gpu, skew) for t in hg]
        out = _dev(torch.zeros(n), gpu, skew)
        sync.aggregate(dg, BATCHES[K], out=out)
        torch.cuda.synchronize()
        want = O.aggregate(hg, BATCHES[K])
        assert torch.equal(_bits(out), _bits(want)), f"K={K} n={n} skew={skew}"


def test_aggregate_in_place_into_vsw0_bucket(gpu):
    from jabas_amd import sync
    K, n = 4, 50001
    hg = _host_grads(K, n, 3)
    dg = [_dev(t, gpu) for t in hg]
    sync.aggregate(dg, BATCHES[K], out=dg[0])
    torch.cuda.synchronize()
    assert torch.equal(_bits(dg[0]), _bits(O.aggregate(hg, BATCHES[K])))
    for k in range(1, K):
        assert torch.equal(_bits(dg[k]), _bits(hg[k]))        # other workers' buckets untouched


def test_aggregate_keeps_zero_rows_exactly_zero(gpu):
    from jabas_amd import sync
    K, rows, cols = 4, 512, 1024
    mask = torch.rand(rows, generator=torch.Generator().manual_seed(0)) < 0.1
    hg = [torch.where(mask[:, None], t.view(rows, cols), torch.zeros(())).reshape(-1)
          for t in _host_grads(K, rows * cols, 5)]
    out = sync.aggregate([_dev(t, gpu) for t in hg], BATCHES[K])
    torch.cuda.synchronize()
    got = out.cpu().view(rows, cols)
    assert torch.all(got[~mask].view(torch.int32) == 0)
    assert torch.equal(_bits(out), _bits(O.aggregate(hg, BATCHES[K])))


# --------------------------------------------------------------------------- statistics
@pytest.mark.parametrize("K", [1, 2, 3, 4, 5, 8, 9, 12, 13, 16])
@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-6), (torch.bfloat16, 1e-2)])
def test_stats_row(gpu, K, dtype, rtol):
    from jabas_amd import sync
    for n, skew in ((5, 0), (4099, 1), (300007, 0), (1 << 21, 2), (4099, 45), (3, 63)):
        print(f"stats K={K} {dtype} n={n} skew={skew}", flush=True)
        hg = _host_grads(K, n, 20 + K, std=5e-4, dtype=dtype)
        row = sync.gradient_stats([_dev(t, gpu, skew) for t in hg], BATCHES[K])
        torch.cuda.synchronize()
        want = O.stats(hg, BATCHES[K])
        got = row.cpu()
        ok, err = _close(got[:4 + K], want[:4 + K], rtol, 1e-30)
        assert ok, f"K={K} n={n}: {got} vs {want}"
        assert torch.count_nonzero(got[4 + K:]) == 0
        # fp64 accumulation (fp32 gradients): in fact far inside the bar; bf16 gradients keep fp32 partial
        # sums over a thread's chunk (products of bf16 values are exact in fp32) and fp64 from there on
        tight = 1e-11 if dtype == torch.float32 else 1e-5
        assert _close(got[1:4 + K], want[1:4 + K], tight, 1e-30)[0], f"K={K} n={n}: {got} vs {want}"
        # the dot product of the halves cancels: its error is measured against |g_A| |g_B| (the cosine's scale)
        assert abs(float(got[0] - want[0])) <= tight * float(torch.sqrt(want[1] * want[2])) + 1e-30


@pytest.mark.parametrize("K", [1, 2, 4, 5, 8, 11, 16])
@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-11), (torch.bfloat16, 1e-5)])
def test_similarity_level_rows(gpu, K, dtype, rtol):
    """Statistics level 2: the four sums of the halves and of the aggregate, per-VSW slots zero; the
    aggregate and an optimizer step in the same launch stay bit-exact."""
    from jabas_amd import sync, _lib as L
    for n, skew in ((5, 0), (4099, 1), (300007, 0), (1 << 21, 2), (4099, 45)):
        print(f"similarity stats K={K} {dtype} n={n} skew={skew}", flush=True)
        hg = _host_grads(K, n, 60 + K, std=5e-4, dtype=dtype)
        dg = [_dev(t, gpu, skew) for t in hg]
        p_h = torch.randn(n, generator=torch.Generator().manual_seed(3)) * 0.05
        m_h, v_h = torch.zeros(n), torch.zeros(n)
        p_d, m_d, v_d, out = _dev(p_h, gpu, skew), _dev(m_h, gpu, skew), _dev(v_h, gpu, skew), _dev(torch.zeros(n), gpu, skew)
        span = sync.SpanSpec(dg, agg_out=out, param=p_d, state1=m_d, state2=v_d)
        args = sync.make_step_args(BATCHES[K], dtype, stats="similarity", opt=ADAMW, step=1)
        assert args.stats == L.STATS_SIMILARITY
        row = sync.sync_bucket(span, args).cpu()
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(hg, BATCHES[K], [(0, n, ())], ADAMW, p_h, m_h, v_h, step=1, want_stats=True)
        assert _close(row[1:4], rows_h[0][1:4], rtol, 1e-30)[0], f"K={K} n={n}: {row[:4]} vs {rows_h[0][:4]}"
        assert abs(float(row[0] - rows_h[0][0])) <= rtol * float(torch.sqrt(rows_h[0][1] * rows_h[0][2])) + 1e-30
        assert torch.count_nonzero(row[4:]) == 0
        assert torch.equal(_bits(out), _bits(agg_h)) and torch.equal(_bits(p_d), _bits(p_h))
        assert torch.equal(_bits(m_d), _bits(m_h)) and torch.equal(_bits(v_d), _bits(v_h))


@pytest.mark.parametrize("K", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("dtype,rtol", [(torch.float32, 1e-11), (torch.bfloat16, 1e-5)])
@pytest.mark.parametrize("opt", [None, SGD, ADAMW], ids=["aggregate", "sgd", "adamw"])
def test_gram_level_rows(gpu, K, dtype, rtol, opt):
    """Statistics level 3: the full row plus the product of every pair of workers, out of the launch that
    aggregates and steps (up to eight workers). Row against the float64
    oracle (the four sums and the norms as at the full level, the pair slots against the Gram matrix), pair order
    as the header's JABAS_STAT_PAIR, slots beyond the row zero, and the aggregate and the optimizer step of the
    same launch bit-exact."""
    from jabas_amd import sync, _lib as L
    for n, skew in ((5, 0), (4099, 1), (300007, 0), (1 << 21, 2), (4099, 45)):
        print(f"gram level K={K} {dtype} n={n} skew={skew}", flush=True)
        hg = _host_grads(K, n, 90 + K, std=5e-4, dtype=dtype)
        dg = [_dev(t, gpu, skew) for t in hg]
        out = _dev(torch.zeros(n), gpu, skew)
        p_h = torch.randn(n, generator=torch.Generator().manual_seed(3)) * 0.05
        m_h, v_h = torch.zeros(n), torch.zeros(n)
        if opt is None:
            span = sync.SpanSpec(dg, agg_out=out)
        else:
            p_d, m_d, v_d = _dev(p_h, gpu, skew), _dev(m_h, gpu, skew), _dev(v_h, gpu, skew)
            span = sync.SpanSpec(dg, agg_out=out, param=p_d, state1=m_d, state2=v_d if opt is ADAMW else None)
        args = sync.make_step_args(BATCHES[K], dtype, stats="gram", opt=opt, step=1, first_step=True)
        assert args.stats == L.STATS_GRAM
        row = sync.sync_bucket(span, args).cpu()
        torch.cuda.synchronize()
        want = O.stats(hg, BATCHES[K])
        G = O.gram(hg)
        width = 4 + K + K * (K - 1) // 2
        assert _close(row[1:4 + K], want[1:4 + K], rtol, 1e-30)[0], f"K={K} n={n}: {row} vs {want}"
        assert abs(float(row[0] - want[0])) <= rtol * float(torch.sqrt(want[1] * want[2])) + 1e-30
        slot = 4 + K
        for a in range(K):
            for b in range(a + 1, K):
                assert L.stat_pair(K, a, b) == slot
                # a pair product cancels: its error is measured against |g_a| |g_b|
                assert abs(float(row[slot] - G[a, b])) <= rtol * float(torch.sqrt(G[a, a] * G[b, b])) + 1e-30, (K, n, a, b)
                slot += 1
        assert slot == width and torch.count_nonzero(row[width:]) == 0
        got = sync.gram_from_stats(row, K)
        assert torch.equal(got, got.t()) and torch.equal(torch.diagonal(got), row[4:4 + K])
        if opt is None:
            assert torch.equal(_bits(out), _bits(O.aggregate(hg, BATCHES[K])))
        else:
            agg_h, _ = O.sync_step(hg, BATCHES[K], [(0, n, ())], opt, p_h, m_h, v_h if opt is ADAMW else None,
                                   step=1, first_step=True, want_stats=False)
            assert torch.equal(_bits(out), _bits(agg_h)) and torch.equal(_bits(p_d), _bits(p_h))
            assert torch.equal(_bits(m_d), _bits(m_h))
            if opt is ADAMW:
                assert torch.equal(_bits(v_d), _bits(v_h))


def test_gram_level_limits_and_the_separate_pass(gpu):
    """More than STATS_GRAM_MAX_K workers are refused before anything is launched; the fused sums agree with
    jabas_gram's own pass over the same buffers (fp32 gradients: both exact products and fp64 sums)."""
    from jabas_amd import sync, _lib as L
    n = 1_000_003
    hg = _host_grads(9, n, 97)
    dg = [_dev(t, gpu, 3) for t in hg]
    out = _dev(torch.zeros(n), gpu, 3)
    before = out.clone()
    with pytest.raises(L.JabasSyncError) as e:
        sync.sync_bucket(sync.SpanSpec(dg, agg_out=out), sync.make_step_args(BATCHES[9], torch.float32, stats="gram"))
    assert e.value.status == L.ERR_K
    assert torch.equal(out, before)
    with pytest.raises(ValueError):
        sync.gram_from_stats(torch.zeros(L.STATS_STRIDE, dtype=torch.float64), 9)
    # the entry point that allocates nothing stops at five workers (its array holds rows of 4 + 16 sums)
    row8 = sync.sync_bucket(sync.SpanSpec(dg[:8], agg_out=out), sync.make_step_args(BATCHES[8], torch.float32, stats="gram"))
    fused8, apart8 = sync.gram_from_stats(row8, 8).cpu(), sync.gram(dg[:8]).cpu()
    scale8 = torch.sqrt(torch.outer(torch.diagonal(apart8), torch.diagonal(apart8)))
    assert bool(((fused8 - apart8).abs() <= 1e-12 * scale8).all())
    hb = _host_grads(9, 70001, 98, std=5e-4, dtype=torch.bfloat16)
    db = [_dev(t, gpu, 3) for t in hb]
    outb = _dev(torch.zeros(70001), gpu, 3)
    with pytest.raises(L.JabasSyncError) as e:
        sync.sync_bucket(sync.SpanSpec(db, agg_out=outb), sync.make_step_args(BATCHES[9], torch.bfloat16, stats="gram"))
    assert e.value.status == L.ERR_K and torch.count_nonzero(outb) == 0
    with pytest.raises(L.JabasSyncError) as e:
        sync.sync_bucket_static(sync.SpanSpec(db[:8], agg_out=outb), sync.make_step_args(BATCHES[8], torch.bfloat16, stats="gram"),
                                stats_out=torch.zeros(L.STATS_STRIDE, dtype=torch.float64, device=gpu))
    assert e.value.status == L.ERR_SIZE and torch.count_nonzero(outb) == 0
    args5 = sync.make_step_args(BATCHES[5], torch.float32, stats="gram")
    row5 = sync.sync_bucket(sync.SpanSpec(dg[:5], agg_out=out), args5).clone()
    row5s = sync.sync_bucket_static(sync.SpanSpec(dg[:5], agg_out=out), args5,
                                    stats_out=torch.zeros(L.STATS_STRIDE, dtype=torch.float64, device=gpu))
    assert torch.equal(row5.cpu().view(torch.int64), row5s.cpu().view(torch.int64)) and float(row5[4 + 5 + 9]) != 0.0
    rowb = sync.sync_bucket(sync.SpanSpec(db[:8], agg_out=outb), sync.make_step_args(BATCHES[8], torch.bfloat16, stats="gram"))
    fusedb, apartb = sync.gram_from_stats(rowb, 8).cpu(), sync.gram(db[:8]).cpu()
    scaleb = torch.sqrt(torch.outer(torch.diagonal(apartb), torch.diagonal(apartb)))
    assert bool(((fusedb - apartb).abs() <= 2e-5 * scaleb).all())
    row = sync.sync_bucket(sync.SpanSpec(dg[:4], agg_out=out), sync.make_step_args(BATCHES[4], torch.float32, stats="gram"))
    fused = sync.gram_from_stats(row, 4).cpu()
    apart = sync.gram(dg[:4]).cpu()
    scale = torch.sqrt(torch.outer(torch.diagonal(apart), torch.diagonal(apart)))
    assert bool(((fused - apart).abs() <= 1e-12 * scale).all())
    again = sync.sync_bucket(sync.SpanSpec(dg[:4], agg_out=out), sync.make_step_args(BATCHES[4], torch.float32, stats="gram"))
    assert torch.equal(again.cpu().view(torch.int64), row.cpu().view(torch.int64))


def test_stats_run_to_run_deterministic(gpu):
    from jabas_amd import sync
    hg = _host_grads(4, 3_000_001, 41)
    dg = [_dev(t, gpu) for t in hg]
    a = sync.gradient_stats(dg, BATCHES[4]).cpu().clone()
    for _ in range(3):
        b = sync.gradient_stats(dg, BATCHES[4]).cpu()
        assert torch.equal(a.view(torch.int64), b.view(torch.int64))


def test_stats_cosine_identities(gpu):
    from jabas_amd import sync
    g0 = _dev(_host_grads(1, 100003, 43)[0], gpu)
    assert sync.cosine_from_stats(sync.gradient_stats([g0, g0.clone()], (8, 8))) == pytest.approx(1.0, abs=1e-12)
    assert sync.cosine_from_stats(sync.gradient_stats([g0, -g0], (8, 8))) == pytest.approx(-1.0, abs=1e-12)
    z = torch.zeros(1000, device=gpu)
    assert sync.cosine_from_stats(sync.gradient_stats([z, z], (1, 1))) == 0.0


@pytest.mark.parametrize("K", list(range(1, 17)))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gram(gpu, K, dtype):
    """fp32 gradients: exact fp64 products and fp64 sums on the vector ALU or the fp64 matrix cores, 1e-11
    against the float64 oracle. bf16 gradients may run on the bf16 matrix cores: exact products, fp32 running
    sums moved into fp64 every few thousand elements, 5e-6 of |g_a| |g_b| against a bar of 1e-2."""
    from jabas_amd import sync
    for n, skew in ((7, 0), (100003, 2), (1 << 20, 0), (100003, 61), (3_000_001, 5)):
        hg = _host_grads(K, n, 30 + K, dtype=dtype)
        G = sync.gram([_dev(t, gpu, skew) for t in hg]).cpu()
        want = O.gram(hg)
        # off-diagonal entries cancel: their error is measured against |g_a| |g_b|
        scale = torch.sqrt(torch.outer(torch.diagonal(want), torch.diagonal(want)))
        off, diag = (1e-12, 1e-11) if dtype == torch.float32 else (5e-6, 5e-6)
        assert bool(((G - want).abs() <= off * scale + 1e-30).all()), f"K={K} n={n}"
        assert _close(torch.diagonal(G), torch.diagonal(want), diag, 1e-30)[0], f"K={K} n={n}"
        assert torch.equal(G, G.t())


def test_gram_limits_and_determinism(gpu):
    from jabas_amd import sync, _lib as L
    g = [torch.zeros(4096, device=gpu) for _ in range(17)]
    with pytest.raises(L.JabasSyncError) as e:
        sync.gram(g)
    assert e.value.status == L.ERR_K
    hg = _host_grads(11, 2_000_003, 77)
    dg = [_dev(t, gpu, 3) for t in hg]
    a = sync.gram(dg).cpu().clone()
    for _ in range(3):
        assert torch.equal(sync.gram(dg).cpu().view(torch.int64), a.view(torch.int64))
    # the diagonal is the per-worker norm row of the statistics kernel's full level
    row = sync.gradient_stats(dg, BATCHES[11]).cpu()
    assert torch.allclose(torch.diagonal(a), row[4:4 + 11], rtol=1e-12, atol=0.0)
    # a workspace without room for the two-stage sum of the partial rows: same values within rounding
    small = torch.empty(1024 * L.GRAM_STRIDE, dtype=torch.float64, device=gpu)
    b = sync.gram(dg, workspace=small).cpu()
    assert torch.allclose(a, b, rtol=1e-13, atol=1e-24)
    with pytest.raises(L.JabasSyncError) as e:
        sync.gram(dg, workspace=small[:1000 * L.GRAM_STRIDE])
    assert e.value.status == L.ERR_WORKSPACE
    hb = _host_grads(13, 1_000_003, 78, dtype=torch.bfloat16)
    db = [_dev(t, gpu, 1) for t in hb]
    a = sync.gram(db).cpu().clone()
    for _ in range(3):
        assert torch.equal(sync.gram(db).cpu().view(torch.int64), a.view(torch.int64))


# ---------------------------------------------------------------------------- optimizer
@pytest.mark.parametrize("hp", [
    dict(lr=0.1, weight_decay=1e-4, momentum=0.9, dampening=0.0, nesterov=False),
    dict(lr=0.05, weight_decay=5e-4, momentum=0.8, dampening=0.0, nesterov=True),
    dict(lr=0.05, weight_decay=1e-3, momentum=0.7, dampening=0.3, nesterov=False),
    dict(lr=0.3, weight_decay=1e-2, momentum=0.0, dampening=0.0, nesterov=False),
])
def test_sgd_steps(gpu, hp):
    from jabas_amd import sync
    n, steps = 70001, 4
    p_h, buf_h = _host_state(n, 1), torch.zeros(n)
    p_d, buf_d = _dev(p_h, gpu), _dev(buf_h, gpu)
    for s in range(steps):
        g = _host_grads(1, n, 50 + s)[0]
        O.sgd_step(p_h, g, buf_h, first_step=(s == 0), **hp)
        sync.sgd_step(_dev(g, gpu), p_d, buf_d if hp["momentum"] else None, first_step=(s == 0), **hp)
        torch.cuda.synchronize()
        ok, err = _close(p_d, p_h, 1e-6, 1e-9)
        assert ok, f"step {s}: max err {err}"
        if hp["momentum"]:
            assert _close(buf_d, buf_h, 1e-6, 2e-9)[0]
    same, tot = _same_bits(p_d, p_h)
    print(f"sgd {hp}: {same}/{tot} weights bit-identical after {steps} steps")
    assert same == tot


@pytest.mark.parametrize("hp", [
    dict(lr=5e-4, weight_decay=0.05, betas=(0.9, 0.999), eps=1e-8, adamw=True),
    dict(lr=2e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, adamw=False),
    dict(lr=1e-3, weight_decay=1e-2, betas=(0.8, 0.99), eps=1e-6, adamw=False),
])
def test_adam_steps(gpu, hp):
    from jabas_amd import sync
    n, steps = 70001, 5
    p_h, m_h, v_h = _host_state(n, 3), torch.zeros(n), torch.zeros(n)
    p_d, m_d, v_d = _dev(p_h, gpu), _dev(m_h, gpu), _dev(v_h, gpu)
    for s in range(1, steps + 1):
        g = _host_grads(1, n, 70 + s, std=5e-4)[0]
        O.adam_step(p_h, g, m_h, v_h, step=s, **hp)
        sync.adam_step(_dev(g, gpu), p_d, m_d, v_d, step=s, **hp)
        torch.cuda.synchronize()
        assert _close(p_d, p_h, 1e-6, 1e-9)[0], f"step {s}"
        assert _close(m_d, m_h, 1e-6, 2e-10)[0], f"step {s}"
        assert _close(v_d, v_h, 1e-6, 1e-16)[0], f"step {s}"
    for name, a, b in (("p", p_d, p_h), ("m", m_d, m_h), ("v", v_d, v_h)):
        same, tot = _same_bits(a, b)
        print(f"adam {hp} {name}: {same}/{tot} bit-identical after {steps} steps")
        assert same == tot


@pytest.mark.parametrize("hp", [
    dict(lr=5e-4, weight_decay=0.05, betas=(0.9, 0.999), eps=1e-8, adamw=True),
    dict(lr=2e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-8, adamw=False),
    dict(lr=1e-3, weight_decay=1e-2, betas=(0.8, 0.99), eps=1e-6, adamw=False),
])
def test_amsgrad_steps(gpu, hp):
    """Adam / AdamW with amsgrad (examples/gnmt/seq2seq/train/shard_optimizer.py:58-66,79-90): weights, both
    moments and the running maximum bit-identical to the oracle over six steps whose gradients shrink after
    the second, so that the maximum and the moment part ways; a NaN gradient element poisons its maximum."""
    from jabas_amd import sync
    n, steps = 70001, 6
    p_h, m_h, v_h, x_h = _host_state(n, 3), torch.zeros(n), torch.zeros(n), torch.zeros(n)
    p_d, m_d, v_d, x_d = _dev(p_h, gpu), _dev(m_h, gpu), _dev(v_h, gpu), _dev(x_h, gpu)
    for s in range(1, steps + 1):
        g = _host_grads(1, n, 170 + s, std=5e-3 if s <= 2 else 2e-4)[0]
        if s == steps:
            g[12345] = float("nan")
        O.adam_step(p_h, g, m_h, v_h, step=s, vmax=x_h, **hp)
        sync.adam_step(_dev(g, gpu), p_d, m_d, v_d, step=s, max_exp_avg_sq=x_d, **hp)
        torch.cuda.synchronize()
        for name, a, b in (("p", p_d, p_h), ("m", m_d, m_h), ("v", v_d, v_h), ("max", x_d, x_h)):
            a = a.detach().cpu()
            nan = torch.isnan(b)                            # (a NaN's payload is not part of the contract)
            assert torch.equal(torch.isnan(a), nan) and int(nan.sum()) == (1 if s == steps else 0), (s, name)
            same, tot = _same_bits(a[~nan], b[~nan])
            assert same == tot, (s, name, same, tot)
    assert float((x_h > v_h).float().mean()) > 0.5 and bool(torch.isnan(x_d[12345])) and bool(torch.isnan(p_d[12345]))


@pytest.mark.parametrize("K,dtype,kind,stats", [(3, torch.float32, "adam", "full"), (8, torch.bfloat16, "adamw", "similarity"),
                                                (4, torch.float32, "adamw", False), (16, torch.bfloat16, "adam", "full"),
                                                (9, torch.float32, "adamw", "similarity")])
def test_sync_bucket_fused_amsgrad(gpu, K, dtype, kind, stats):
    """The fused launch with the amsgrad kinds: aggregate, statistics, weights, moments, maximum and the
    replica all from one pass, bit-identical to the oracle (statistics within their bar)."""
    from jabas_amd import sync
    n = 200003
    skew = 3 if dtype == torch.bfloat16 else 1
    bounds = ((0, 1), (5, 0), (1029, 1), (70000, 0), (70001, 1), (150000, 0))
    opt = dict(ADAMW if kind == "adamw" else ADAM, amsgrad=True)
    p_h, s1_h, s2_h, s3_h = _host_state(n, 5), torch.zeros(n), torch.zeros(n), torch.zeros(n)
    agg_d = _dev(torch.zeros(n), gpu, skew)
    p_d, s1_d, s2_d, s3_d = (_dev(t, gpu, skew) for t in (p_h, s1_h, s2_h, s3_h))
    fan = [_dev(torch.zeros(n), gpu, skew)]
    dg = [_dev(torch.zeros(n, dtype=dtype), gpu, skew) for _ in range(K)]
    span = sync.SpanSpec(dg, agg_out=agg_d, param=p_d, state1=s1_d, state2=s2_d, state3=s3_d, fanout=fan, bounds=bounds)
    ws = sync.Workspace.for_span(n, dtype, gpu)
    for step in (1, 2, 3, 4):
        hg = _host_grads(K, n, 460 + K + step, std=5e-3 if step <= 2 else 2e-4, dtype=dtype)
        for d, h in zip(dg, hg):
            d.copy_(h)
        args = sync.make_step_args(BATCHES[K], dtype, stats=stats, opt=opt, step=step)
        row = sync.sync_bucket(span, args, workspace=ws)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(hg, BATCHES[K], [(0, n, bounds)], opt, p_h, s1_h, s2_h, step=step,
                                    want_stats=bool(stats), state3=s3_h)
        assert torch.equal(_bits(agg_d), _bits(agg_h)), f"step {step}"
        for name, a, b in (("p", p_d, p_h), ("m", s1_d, s1_h), ("v", s2_d, s2_h), ("max", s3_d, s3_h), ("replica", fan[0], p_h)):
            same, tot = _same_bits(a, b)
            assert same == tot, (step, name, same, tot)
        if stats:
            rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
            width = 4 + K if stats == "full" else 4
            assert _close(row.cpu()[1:width], rows_h[0][1:width], rtol, 1e-30)[0]
            assert abs(float(row[0].cpu() - rows_h[0][0])) <= rtol * float(torch.sqrt(rows_h[0][1] * rows_h[0][2]))
    assert float((s3_h > s2_h).float().mean()) > 0.1          # the maximum did part from the moment


@pytest.mark.parametrize("K,dtype,kind,stats,amsgrad", [
    (4, torch.float32, "adamw", "similarity", False), (8, torch.bfloat16, "adamw", "similarity", False),
    (8, torch.bfloat16, "adamw", False, False), (2, torch.float32, "adam", "full", True),
    (8, torch.bfloat16, "adam", "full", True), (3, torch.float32, "adamw", "gram", False),
    (12, torch.float32, "adam", False, False), (1, torch.float32, "adamw", False, True)])
@pytest.mark.parametrize("block_log2", [8, 11, 13])
def test_interleaved_moments(gpu, K, dtype, kind, stats, amsgrad, block_log2):
    """Adam's moments in one arena of alternating blocks (JabasSpan.state_block_log2): spans that start at
    arbitrary elements of the arena, in the middle of a block, shorter than a block and across many blocks, with
    parameter-group bounds and element skews; aggregate, weights and every moment bit-identical to the oracle's
    flat arrays, nothing of the arena outside the span's own elements touched."""
    from jabas_amd import sync
    opt = dict(ADAMW if kind == "adamw" else ADAM, amsgrad=amsgrad)
    ways, T = (3 if amsgrad else 2), 1 << block_log2
    total = 5 * T + 70001
    arena = sync.MomentArena(total, ways, gpu, block_log2)
    marker = 7.25
    arena.buf.fill_(marker)
    cases = [(0, 4099, 0), (T - 64, 3 * T + 200, 0), (T + 320, 37, 0), (2 * T + 64 * 5 + 3, 70001, 3), (4 * T - 4 + 1, 2 * T, 1)]
    for ci, (first, n, skew) in enumerate(cases):
        skew = first % 64                          # every buffer of a span sits at the same element of a 256-byte line
        print(f"interleaved K={K} {dtype} T={T} first={first} n={n}", flush=True)
        bounds = ((0, 1), (5, 0), (min(1029, n - 1), 1)) if n > 1100 else ((0, 0),)
        p_h = _host_state(n, 5 + ci)
        m_h, v_h, x_h = torch.zeros(n), torch.zeros(n), torch.zeros(n)
        for j in range(ways):
            arena.write(j, torch.zeros(n, device=gpu), first)
        agg_d = _dev(torch.zeros(n), gpu, skew)
        p_d = _dev(p_h, gpu, skew)
        dg = [_dev(torch.zeros(n, dtype=dtype), gpu, skew) for _ in range(K)]
        span = sync.SpanSpec(dg, agg_out=agg_d, param=p_d, bounds=bounds, moments=(arena, first))
        ws = sync.Workspace.for_span(n, dtype, gpu)
        for step in (1, 2, 3):
            hg = _host_grads(K, n, 700 + K + step + ci, std=5e-3 if step <= 2 else 2e-4, dtype=dtype)
            for d, h in zip(dg, hg):
                d.copy_(h)
            row = sync.sync_bucket(span, sync.make_step_args(BATCHES[K], dtype, stats=stats, opt=opt, step=step), workspace=ws)
            torch.cuda.synchronize()
            agg_h, rows_h = O.sync_step(hg, BATCHES[K], [(0, n, bounds)], opt, p_h, m_h, v_h, step=step,
                                        want_stats=bool(stats), state3=x_h if amsgrad else None)
            assert torch.equal(_bits(agg_d), _bits(agg_h)), (first, step)
            got = [arena.read(j, first, n) for j in range(ways)]
            for name, a, b in (("p", p_d, p_h), ("m", got[0], m_h), ("v", got[1], v_h)) + ((("max", got[2], x_h),) if amsgrad else ()):
                same, tot = _same_bits(a, b)
                assert same == tot, (first, n, step, name, same, tot)
            if stats:
                rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
                assert _close(row.cpu()[1:4], rows_h[0][1:4], rtol, 1e-30)[0]
    # what the spans did not own still holds the marker
    owned = torch.zeros(arena.blocks * T, dtype=torch.bool, device=gpu)
    for first, n, _ in cases:
        owned[first:first + n] = True
    for j in range(ways):
        rest = arena.way(j).reshape(-1)[~owned]
        assert bool((rest == marker).all()), j


def test_interleaved_moments_are_checked(gpu):
    """Layout rules of interleaved moments: Adam kinds only, state2 / state3 whole blocks behind state1, the
    block position inside the block, the block group on a 16-byte line; the moments count as one written range."""
    import ctypes as C
    from jabas_amd import sync, _lib as L
    lib = L.lib()
    n, b = 5000, 10
    T = 1 << b
    arena = sync.MomentArena(8 * T, 2, gpu, b)
    g = [torch.zeros(n, device=gpu)]
    p = torch.zeros(n, device=gpu)
    adam = sync.make_step_args((1,), torch.float32, opt=ADAM, step=1)
    sgd = sync.make_step_args((1,), torch.float32, opt=SGD, first_step=True)

    def call(span, args=adam):
        return lib.jabas_sync_bucket(C.byref(span), None, C.byref(args), None, None, 0, None)
    good = sync.SpanSpec(g, param=p, moments=(arena, 0)).to_c()
    assert call(good) == L.OK
    assert call(good, sgd) == L.ERR_OPT
    bad = sync.SpanSpec(g, param=p, moments=(arena, 0)).to_c()
    bad.state2 = bad.state1 + 4 * T + 16
    assert call(bad) == L.ERR_ALIGN
    bad = sync.SpanSpec(g, param=p, moments=(arena, 0)).to_c()
    bad.state_block_pos = T
    assert call(bad) == L.ERR_SIZE
    bad = sync.SpanSpec(g, param=p, moments=(arena, 0)).to_c()
    bad.state_block_log2 = 7
    assert call(bad) == L.ERR_SIZE
    bad = sync.SpanSpec(g, param=p, moments=(arena, 0)).to_c()
    bad.state_block_pos = 2                                   # the block group would start 8 bytes off a 16-byte line
    assert call(bad) == L.ERR_ALIGN
    # the weights inside the moments' range (the gap between two of the span's blocks is part of that range)
    inside = arena.buf[2 * T:2 * T + n]
    assert call(sync.SpanSpec(g, param=inside, moments=(arena, 0)).to_c()) == L.ERR_ALIAS
    ams = sync.make_step_args((1,), torch.float32, opt=dict(ADAM, amsgrad=True), step=1)
    assert call(good, ams) == L.ERR_NULL                      # two moments interleaved where the optimizer keeps three
    torch.cuda.synchronize()


def test_amsgrad_needs_its_maximum_and_is_not_replayed_from_a_block(gpu):
    from jabas_amd import sync, _lib as L
    n = 4096
    g = [torch.zeros(n, device=gpu)]
    p, m, v = (torch.zeros(n, device=gpu) for _ in range(3))
    opt = dict(ADAM, amsgrad=True)
    args = sync.make_step_args((1,), torch.float32, opt=opt, step=1)
    assert args.opt_kind == L.OPT_ADAM_AMSGRAD
    with pytest.raises(L.JabasSyncError) as e:
        sync.sync_bucket(sync.SpanSpec(g, param=p, state1=m, state2=v), args)
    assert e.value.status == L.ERR_NULL
    with pytest.raises(L.JabasSyncError) as e:
        sync.SyncPlan([sync.SpanSpec(g, param=p, state1=m, state2=v)], L.OPT_ADAMW_AMSGRAD)
    assert e.value.status == L.ERR_NULL
    with pytest.raises(ValueError):
        sync.opt_kind(dict(SGD, amsgrad=True))


# ------------------------------------------------------------------ fused, single bucket
@pytest.mark.parametrize("K,dtype,opt", [(2, torch.float32, SGD), (4, torch.float32, ADAMW),
                                         (3, torch.float32, ADAM), (8, torch.bfloat16, ADAMW),
                                         (5, torch.bfloat16, SGD), (1, torch.float32, ADAM),
                                         (9, torch.float32, ADAM), (12, torch.float32, SGD),
                                         (13, torch.bfloat16, ADAM), (16, torch.bfloat16, ADAMW),
                                         (16, torch.float32, ADAMW)])
def test_sync_bucket_fused(gpu, K, dtype, opt):
    from jabas_amd import sync
    n = 200003
    skew = 3 if dtype == torch.bfloat16 else 1
    bounds = ((0, 1), (5, 0), (1029, 1), (70000, 0), (70001, 1), (150000, 0))
    hg = _host_grads(K, n, 60 + K, std=5e-4, dtype=dtype)
    p_h, s1_h, s2_h = _host_state(n, 5), torch.zeros(n), torch.zeros(n)
    dg = [_dev(t, gpu, skew) for t in hg]
    agg_d = _dev(torch.zeros(n), gpu, skew)
    p_d, s1_d, s2_d = _dev(p_h, gpu, skew), _dev(s1_h, gpu, skew), _dev(s2_h, gpu, skew)
    fan = [_dev(torch.zeros(n), gpu, skew) for _ in range(2)]
    adam = opt["kind"] != "sgd"
    span = sync.SpanSpec(dg, agg_out=agg_d, param=p_d, state1=s1_d, state2=s2_d if adam else None, fanout=fan,
                         bounds=bounds)
    ws = sync.Workspace.for_span(n, dtype, gpu)
    for step in (1, 2, 3):
        args = sync.make_step_args(BATCHES[K], dtype, stats=True, opt=opt, step=step, first_step=(step == 1))
        row = sync.sync_bucket(span, args, workspace=ws)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(hg, BATCHES[K], [(0, n, bounds)], opt, p_h, s1_h, s2_h if adam else None,
                                    step=step, first_step=(step == 1), want_stats=True)
        assert torch.equal(_bits(agg_d), _bits(agg_h)), f"step {step}"
        rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
        assert _close(row.cpu()[:4 + K], rows_h[0][:4 + K], rtol, 1e-30)[0]
        assert _close(p_d, p_h, 1e-6, 1e-9)[0], f"step {step}"
        assert _close(s1_d, s1_h, 1e-6, 2e-9)[0], f"step {step}"
        if adam:
            assert _close(s2_d, s2_h, 1e-6, 1e-16)[0], f"step {step}"
        for f in fan:
            assert torch.equal(_bits(f), _bits(p_d))
    same, tot = _same_bits(p_d, p_h)
    print(f"fused bucket K={K} {dtype} {opt['kind']}: {same}/{tot} weights bit-identical")
    assert same == tot


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("skews", [
    "37 for every buffer",                # one offset within 256 bytes: the launch's element grid starts at that line
    "differs within 256 bytes",           # equal only within 16 bytes: the grid starts at the first element's 16-byte line
    "63 for every buffer", "60 for every buffer"])
def test_sync_bucket_buffer_offsets_within_a_256_byte_line(gpu, dtype, skews):
    """Where the launch's element grid starts depends on how the buffers sit relative to 256-byte
    lines; the results must not."""
    from jabas_amd import sync
    K, n = 3, 150001
    bounds = ((0, 1), (3, 0), (61, 1), (1024, 0), (99999, 1))
    if skews.endswith("for every buffer"):
        sk = [int(skews.split()[0])] * 8
    else:
        sk = [5, 9, 61, 33, 1, 17, 49, 13]             # all 1 mod 4
    hg = _host_grads(K, n, 300, std=5e-4, dtype=dtype)
    p_h, s1_h, s2_h = _host_state(n, 6), torch.zeros(n), torch.zeros(n)
    dg = [_dev(t, gpu, sk[k]) for k, t in enumerate(hg)]
    agg_d = _dev(torch.zeros(n), gpu, sk[3])
    p_d, s1_d, s2_d = _dev(p_h, gpu, sk[4]), _dev(s1_h, gpu, sk[5]), _dev(s2_h, gpu, sk[6])
    fan = [_dev(torch.zeros(n), gpu, sk[7])]
    guard = [t._base if t._base is not None else t for t in dg + [agg_d, p_d, s1_d, s2_d] + fan]
    before = [(b[:sk_i].clone(), b[sk_i + n:].clone()) for b, sk_i in zip(guard, sk)]
    span = sync.SpanSpec(dg, agg_out=agg_d, param=p_d, state1=s1_d, state2=s2_d, fanout=fan, bounds=bounds)
    ws = sync.Workspace.for_span(n, dtype, gpu)
    for step in (1, 2):
        args = sync.make_step_args(BATCHES[K], dtype, stats=True, opt=ADAMW, step=step, first_step=(step == 1))
        row = sync.sync_bucket(span, args, workspace=ws)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(hg, BATCHES[K], [(0, n, bounds)], ADAMW, p_h, s1_h, s2_h, step=step,
                                    first_step=(step == 1), want_stats=True)
        assert torch.equal(_bits(agg_d), _bits(agg_h)), step
        rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
        assert _close(row.cpu()[:4 + K], rows_h[0][:4 + K], rtol, 1e-30)[0]
        for got, want in ((p_d, p_h), (s1_d, s1_h), (s2_d, s2_h), (fan[0], p_h)):
            assert torch.equal(_bits(got), _bits(want)), step
    # nothing outside the live range was written
    for b, sk_i, (head, tail) in zip(guard, sk, before):
        assert torch.equal(b[:sk_i], head) and torch.equal(b[sk_i + n:], tail)


# ---------------------------------------------------------------- fused, multi-span plan
@pytest.mark.parametrize("K,dtype,opt,in_place", [
    (2, torch.float32, SGD, True), (4, torch.float32, ADAMW, True), (3, torch.float32, SGD, False),
    (4, torch.float32, ADAM, False), (8, torch.bfloat16, ADAMW, False), (6, torch.float32, None, True),
    (7, torch.bfloat16, None, False), (10, torch.float32, ADAMW, True), (16, torch.bfloat16, SGD, False),
    (15, torch.float32, None, False)])
def test_sync_fused_plan_ragged_spans(gpu, K, dtype, opt, in_place):
    from jabas_amd import sync, _lib as L
    # span sizes: tiny, exactly one tile, ragged, empty, large; offsets chosen so that some
    # spans start off a 16-byte line (all buffers share the offset, as views of one layout do)
    sizes = [1, 1024, 2048, 0, 4097, 333, 8192 * 3 + 5, 7, 500000, 64, 2048 * 40]
    gaps = [0, 3, 0, 1, 0, 2, 0, 0, 5, 0, 0]
    offs, off = [], 0
    for s, gp in zip(sizes, gaps):
        off += gp
        offs.append(off)
        off += s
    total = off
    hg = _host_grads(K, total, 80 + K, std=5e-4, dtype=dtype)
    p_h, s1_h, s2_h = _host_state(total, 7), torch.zeros(total), torch.zeros(total)
    dg = [_dev(t, gpu) for t in hg]
    agg_d = dg[0] if in_place else _dev(torch.zeros(total), gpu)
    p_d, s1_d, s2_d = _dev(p_h, gpu), _dev(s1_h, gpu), _dev(s2_h, gpu)
    kind = sync.opt_kind(opt)
    adam = kind in (L.OPT_ADAM, L.OPT_ADAMW)
    spans_h, spans_d = [], []
    for i, (o, s) in enumerate(zip(offs, sizes)):
        if s > 3000:
            bounds = ((0, i % 2), (s // 3, 1 - i % 2), (s // 3 + 1, i % 2), (s - 1, 1))
        elif s > 0:
            bounds = ((0, i % 2),)
        else:
            bounds = ()
        sl = slice(o, o + s)
        spans_h.append((o, s, bounds))
        spans_d.append(sync.SpanSpec([g[sl] for g in dg], agg_out=agg_d[sl],
                                     param=p_d[sl] if opt else None, state1=s1_d[sl] if opt else None,
                                     state2=s2_d[sl] if adam else None, bounds=bounds if opt else ()))
    plan = sync.SyncPlan(spans_d, kind)
    hg_work = [t.clone() for t in hg]
    for step in (1, 2):
        args = sync.make_step_args(BATCHES[K], dtype, stats=True, opt=opt, step=step, first_step=(step == 1))
        rows = plan.run(args)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(hg_work, BATCHES[K], spans_h, opt, p_h, s1_h, s2_h if adam else None,
                                    step=step, first_step=(step == 1), want_stats=True)
        for (o, s, _), i in zip(spans_h, range(len(spans_h))):
            assert torch.equal(_bits(agg_d[o:o + s]), _bits(agg_h[o:o + s])), f"span {i} step {step}"
        rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
        ok, err = _close(rows.cpu()[:, :4 + K], rows_h[:, :4 + K], rtol, 1e-30)
        assert ok, f"stats step {step}: {rows.cpu()} vs {rows_h}"
        if opt:
            assert _close(p_d, p_h, 1e-6, 1e-9)[0], f"step {step}"
            assert _close(s1_d, s1_h, 1e-6, 2e-9)[0]
            if adam:
                assert _close(s2_d, s2_h, 1e-6, 1e-16)[0]
        if in_place:
            # the next step aggregates what is now in VSW 0's buckets, on both sides
            for (o, s, _) in spans_h:
                hg_work[0][o:o + s] = agg_h[o:o + s]
    # elements in the gaps between spans are never written
    covered = torch.zeros(total, dtype=torch.bool)
    for o, s, _ in spans_h:
        covered[o:o + s] = True
    if opt:
        assert torch.equal(_bits(p_d)[~covered], _bits(_host_state(total, 7))[~covered])


def test_fused_rejects_bad_arguments(gpu):
    from jabas_amd import sync, _lib as L
    n = 4096
    g = [torch.zeros(n + 8, device=gpu) for _ in range(2)]
    out = torch.zeros(n + 8, device=gpu)
    with pytest.raises(L.JabasSyncError) as e:
        sync.aggregate([g[0][1:n + 1], g[1][:n]], (1, 1), out=out[:n])       # mutually misaligned
    assert e.value.status == L.ERR_ALIGN
    with pytest.raises(L.JabasSyncError) as e:
        sync.aggregate([g[0][:n], g[1][:n]], (1, 1), out=g[0][4:n + 4])      # partial overlap
    assert e.value.status == L.ERR_ALIAS
    with pytest.raises(ValueError):
        sync.aggregate([g[0][:n]] * 17, (1,) * 17)
    span = sync.SpanSpec([g[0][:n], g[1][:n]], param=None)
    args = sync.make_step_args((1, 1), torch.float32, opt=SGD)
    with pytest.raises(L.JabasSyncError) as e:
        sync.sync_bucket(span, args)                                          # optimizer without weights
    assert e.value.status == L.ERR_NULL


def test_span_beyond_two_to_the_31_elements(gpu):
    """64-bit element indexing: one span of 2^31 + 4099 elements (8.6 GB per buffer)."""
    from jabas_amd import sync
    n = (1 << 31) + 4099
    g0 = torch.empty(n, dtype=torch.float32, device=gpu)
    g1 = torch.empty(n, dtype=torch.float32, device=gpu)
    step = 1 << 27
    for lo in range(0, n, step):                       # value depends on the position, cheap to regenerate
        hi = min(n, lo + step)
        idx = torch.arange(lo, hi, device=gpu, dtype=torch.int64)
        g0[lo:hi] = ((idx % 1021).float() - 510.0) * 2.0 ** -10
        g1[lo:hi] = ((idx % 4093).float() - 2046.0) * 2.0 ** -12
        del idx
    out = torch.empty(n, dtype=torch.float32, device=gpu)
    sync.aggregate([g0, g1], (1, 1), out=out)          # weights 0.5, 0.5: every product and the sum are exact
    row = sync.gradient_stats([g0, g1], (1, 1)).cpu()
    torch.cuda.synchronize()
    norm0 = 0.0
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        want = g0[lo:hi] * 0.5 + g1[lo:hi] * 0.5
        assert torch.equal(out[lo:hi].view(torch.int32), want.view(torch.int32)), lo
        norm0 += float((g0[lo:hi].double() ** 2).sum())
        del want
    assert float(row[4]) == pytest.approx(norm0, rel=1e-10)


def test_special_values_denormals_infinities_nans(gpu):
    """Denormal inputs and results are kept (no flush to zero), infinities and NaNs stay in
    the element they entered, signed zeros follow IEEE addition."""
    from jabas_amd import sync
    K, n = 3, 5000
    hg = _host_grads(K, n, 99)
    hg[0][:64] = torch.logspace(-45, -38, 64)                 # denormal inputs
    hg[1][:64] = -torch.logspace(-44.5, -38.2, 64)
    hg[2][:64] = 0.0
    hg[0][100], hg[1][101], hg[2][102] = float("inf"), float("-inf"), float("nan")
    hg[0][103], hg[1][103] = float("inf"), float("-inf")       # inf - inf -> nan
    hg[0][200:210], hg[1][200:210], hg[2][200:210] = -0.0, -0.0, -0.0
    hg[0][210:220], hg[1][210:220], hg[2][210:220] = -0.0, 0.0, -0.0
    out = sync.aggregate([_dev(t, gpu) for t in hg], BATCHES[K]).cpu()
    want = O.aggregate(hg, BATCHES[K])
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(out), nan) and int(nan.sum()) == 2
    assert torch.equal(out[~nan].view(torch.int32), want[~nan].view(torch.int32))
    assert torch.count_nonzero(out[:64]) > 32                  # denormal results survived
    assert torch.all(out[200:210].view(torch.int32) == torch.tensor(-0.0).view(torch.int32))
    assert torch.all(out[210:220].view(torch.int32) == 0)
    # Adam on a gradient whose square is denormal: v stays denormal, the step is still the sign step
    g = torch.full((2048,), 1e-21)
    p_h, m_h, v_h = torch.ones(2048), torch.zeros(2048), torch.zeros(2048)
    p_d, m_d, v_d = _dev(p_h, gpu), _dev(m_h, gpu), _dev(v_h, gpu)
    hp = dict(lr=1e-3, weight_decay=0.0, betas=(0.9, 0.999), eps=1e-30, adamw=False)
    O.adam_step(p_h, g, m_h, v_h, step=1, **hp)
    sync.adam_step(_dev(g, gpu), p_d, m_d, v_d, step=1, **hp)
    torch.cuda.synchronize()
    assert 0 < float(v_h[0]) < 1.2e-38                         # denormal second moment
    for a, b in ((p_d, p_h), (m_d, m_h), (v_d, v_h)):
        assert torch.equal(_bits(a), _bits(b))


# ------------------------------------------------------------- randomized plans vs the oracle
def _random_case(seed):
    rng = np.random.RandomState(seed)
    K = int(rng.randint(1, 9)) if seed < 16 else int(rng.randint(9, 17))
    dtype = torch.bfloat16 if rng.rand() < 0.4 else torch.float32
    opt = [None, SGD, ADAM, ADAMW][int(rng.randint(0, 4))]
    if opt is SGD and rng.rand() < 0.3:
        opt = dict(SGD, nesterov=True, momentum=0.8)
    n_span = int(rng.randint(1, 25))
    sizes = []
    for _ in range(n_span):
        kind = rng.rand()
        if kind < 0.1:
            sizes.append(0)
        elif kind < 0.5:
            sizes.append(int(rng.randint(1, 3000)))
        elif kind < 0.8:
            sizes.append(int(1024 * rng.randint(1, 9) + rng.choice([-1, 0, 1, 2])))
        else:
            sizes.append(int(rng.randint(20000, 120000)))
    gaps = [int(rng.randint(0, 9)) for _ in sizes]
    half_id = None
    if K >= 2 and rng.rand() < 0.5:                      # arbitrary halves, both non-empty
        while True:
            half_id = [int(v) for v in rng.randint(0, 2, size=K)]
            if 0 < sum(half_id) < K:
                break
    batches = tuple(int(v) for v in rng.randint(1, 65, size=K))
    in_place = dtype == torch.float32 and rng.rand() < 0.5
    n_fan = int(rng.randint(0, 3)) if opt else 0
    bounds = []
    for s in sizes:
        if opt is None or s == 0:
            bounds.append(())
            continue
        nb = int(rng.randint(0, 5))
        starts = sorted(set([0] + [int(v) for v in rng.randint(1, max(2, s), size=nb) if v < s]))
        bounds.append(tuple((st, int(rng.randint(0, 2))) for st in starts))
    return K, dtype, opt, sizes, gaps, half_id, batches, in_place, n_fan, bounds


@pytest.mark.parametrize("seed", range(24))
def test_random_plans_match_the_oracle(gpu, seed):
    """Random K, dtype, optimizer, span sizes (empty, sub-tile, tile-edge, large), line offsets, group
    bounds, halves, fan-out and in-place aggregation: the planned launch against the oracle over 3 steps."""
    from jabas_amd import sync, _lib as L
    K, dtype, opt, sizes, gaps, half_id, batches, in_place, n_fan, bounds = _random_case(seed)
    print(f"seed {seed}: K={K} {dtype} opt={opt and opt['kind']} spans={sizes} gaps={gaps} halves={half_id} "
          f"in_place={in_place} fan={n_fan}", flush=True)
    offs, off = [], 0
    for s, gp in zip(sizes, gaps):
        off += gp
        offs.append(off)
        off += s
    total = max(off, 1)
    hg = _host_grads(K, total, 300 + seed, std=5e-4, dtype=dtype)
    p_h, s1_h, s2_h = _host_state(total, 40 + seed), torch.zeros(total), torch.zeros(total)
    base_skew = seed % 4
    srng = np.random.RandomState(7000 + seed)

    def skew():
        """Every third seed puts each buffer at its own place of a 256-byte line (equal within 16
        bytes only: the launch falls back to the 16-byte element grid); the others share one place."""
        return base_skew + (4 * int(srng.randint(0, 16)) if seed % 3 == 2 else 4 * (seed % 16))
    dg = [_dev(t, gpu, skew()) for t in hg]
    agg_d = dg[0] if in_place else _dev(torch.zeros(total), gpu, skew())
    p_d, s1_d, s2_d = _dev(p_h, gpu, skew()), _dev(s1_h, gpu, skew()), _dev(s2_h, gpu, skew())
    fans = [_dev(torch.zeros(total), gpu, skew()) for _ in range(n_fan)]
    kind = sync.opt_kind(opt)
    adam = kind in (L.OPT_ADAM, L.OPT_ADAMW)
    # every other Adam case keeps the moments interleaved in one arena (blocks of 256, 1024 or 8192 elements), the
    # arena's element 0 at the weights' place of a 16-byte line (of a 256-byte line when all buffers share one)
    arena = None
    if adam and seed % 4 >= 2:
        arena_first = skew()
        arena = sync.MomentArena(arena_first + total, 2, gpu, (8, 10, 13)[seed % 3])
    spans_h, spans_d = [], []
    for o, s, b in zip(offs, sizes, bounds):
        sl = slice(o, o + s)
        spans_h.append((o, s, b))
        state = dict(moments=(arena, arena_first + o)) if arena is not None else \
            dict(state1=s1_d[sl] if opt else None, state2=s2_d[sl] if adam else None)
        spans_d.append(sync.SpanSpec([g[sl] for g in dg], agg_out=agg_d[sl], param=p_d[sl] if opt else None,
                                     fanout=[f[sl] for f in fans], bounds=b, **state))
    plan = sync.SyncPlan(spans_d, kind)
    hg_work = [t.clone() for t in hg]
    block = sync.StepScalars(gpu) if opt and seed % 2 else None
    for step in (1, 2, 3):
        # full rows on the first step, none on the second; on the third the similarity sums or, up to eight
        # workers, the full rows with the pair products
        stats = (True, False, "gram" if K <= L.STATS_GRAM_MAX_K and seed % 3 else "similarity")[step - 1]
        args = sync.make_step_args(batches, dtype, stats=stats, opt=opt, step=step, first_step=(step == 1),
                                   half_id=half_id)
        if block is not None:
            # odd seeds: the step's scalars travel in the device block; the by-value arguments of the call are
            # those of another step at another learning rate, as in a launch recorded once and replayed
            block.update(args)
            args = block.attach(sync.make_step_args(batches, dtype, stats=stats, opt=opt, step=5, first_step=(step != 1),
                                                    half_id=half_id, lr_scale=3.0))
        rows = plan.run(args)
        torch.cuda.synchronize()
        hg_in = [t.clone() for t in hg_work]            # what this step's launch read (the in-place aggregate moves worker 0's)
        agg_h, rows_h = O.sync_step(hg_work, batches, spans_h, opt, p_h, s1_h, s2_h if adam else None, step=step,
                                    first_step=(step == 1), want_stats=bool(stats), half_id=half_id)
        for i, (o, s, _) in enumerate(spans_h):
            assert torch.equal(_bits(agg_d[o:o + s]), _bits(agg_h[o:o + s])), f"span {i} step {step}"
        if stats:
            rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
            width = 4 if stats == "similarity" else 4 + K
            got, want = rows.cpu()[:, :width], rows_h[:, :width]
            scale = want[:, 1:3].abs().max(dim=1, keepdim=True).values.clamp_min(1e-300)   # dot may cancel: bound it by the norms
            assert bool(((got - want).abs() <= rtol * want.abs() + 1e-9 * scale).all()), f"stats step {step}"
            pairs = K * (K - 1) // 2 if stats == "gram" else 0
            assert torch.count_nonzero(rows[:, width + pairs:]) == 0
            if pairs:
                for i, (o, sz, _) in enumerate(spans_h):
                    G = O.gram([t[o:o + sz] for t in hg_in])
                    for a in range(K):
                        for b in range(a + 1, K):
                            err = abs(float(rows[i, L.stat_pair(K, a, b)]) - float(G[a, b]))
                            assert err <= (1e-5 if dtype == torch.bfloat16 else 1e-11) * float(torch.sqrt(G[a, a] * G[b, b])) + 1e-300, \
                                f"pair ({a}, {b}) span {i}"
        if opt:
            if arena is not None:
                s1_d, s2_d = arena.read(0, arena_first, total), arena.read(1, arena_first, total)
            for i, (o, s, _) in enumerate(spans_h):
                assert torch.equal(_bits(p_d[o:o + s]), _bits(p_h[o:o + s])), f"weights span {i} step {step}"
                assert torch.equal(_bits(s1_d[o:o + s]), _bits(s1_h[o:o + s])), f"state1 span {i} step {step}"
                if adam:
                    assert torch.equal(_bits(s2_d[o:o + s]), _bits(s2_h[o:o + s])), f"state2 span {i} step {step}"
                for f in fans:
                    assert torch.equal(_bits(f[o:o + s]), _bits(p_d[o:o + s]))
        if in_place:
            for (o, s, _) in spans_h:
                hg_work[0][o:o + s] = agg_h[o:o + s]
    # nothing outside the spans was written
    covered = torch.zeros(total, dtype=torch.bool)
    for o, s, _ in spans_h:
        covered[o:o + s] = True
    if opt and (~covered).any():
        assert torch.equal(_bits(p_d)[~covered], _bits(_host_state(total, 40 + seed))[~covered])
        if arena is not None:                                # the moments of elements no span owns stayed zero
            assert torch.count_nonzero(arena.read(0, arena_first, total)[~covered.to(gpu)]) == 0
            assert torch.count_nonzero(arena.read(1, arena_first, total)[~covered.to(gpu)]) == 0
        for f in fans:
            assert torch.count_nonzero(f.cpu()[~covered]) == 0
    if not in_place and (~covered).any():
        assert torch.count_nonzero(agg_d.cpu()[~covered]) == 0


@pytest.mark.parametrize("seed", list(range(100, 112)) + [116, 117, 119, 121])
def test_random_buckets_through_the_inline_path(gpu, seed):
    """The same random cases, one jabas_sync_bucket call per span (span by value, bound table on the
    device, first bound of each workgroup found by binary search)."""
    from jabas_amd import sync, _lib as L
    K, dtype, opt, sizes, gaps, half_id, batches, in_place, n_fan, bounds = _random_case(seed - 100 if seed % 2 else seed)
    rng = np.random.RandomState(seed)
    sizes = [s for s in sizes if s > 0][:8] or [777]
    bounds = [b for s, b in zip(sizes, [b for b in bounds if b] + [()] * len(sizes))]
    print(f"seed {seed}: K={K} {dtype} opt={opt and opt['kind']} sizes={sizes} halves={half_id}", flush=True)
    kind = sync.opt_kind(opt)
    adam = kind in (L.OPT_ADAM, L.OPT_ADAMW)
    for si, n in enumerate(sizes):
        skew = int(rng.randint(0, 4))
        b = tuple((st, g) for st, g in bounds[si] if st < n) if opt else ()
        if opt and (not b or b[0][0] != 0):
            b = ((0, 1),) + tuple(x for x in b if x[0] > 0)
        hg = _host_grads(K, n, 500 + 13 * seed + si, std=5e-4, dtype=dtype)
        p_h, s1_h, s2_h = _host_state(n, 60 + seed + si), torch.zeros(n), torch.zeros(n)
        dg = [_dev(t, gpu, skew) for t in hg]
        agg_d = _dev(torch.zeros(n), gpu, skew)
        p_d, s1_d, s2_d = _dev(p_h, gpu, skew), _dev(s1_h, gpu, skew), _dev(s2_h, gpu, skew)
        span = sync.SpanSpec(dg, agg_out=agg_d, param=p_d if opt else None, state1=s1_d if opt else None,
                             state2=s2_d if adam else None, bounds=b)
        call = sync.BucketCall(span)
        block = sync.StepScalars(gpu) if opt and (seed + si) % 2 else None
        for step in (1, 2, 3):
            stats = step != 2                  # the plain launch may run another workgroup shape
            args = sync.make_step_args(batches, dtype, stats=stats, opt=opt, step=step, first_step=(step == 1),
                                       half_id=half_id)
            if block is not None:              # every other bucket: scalars from the device block, stale ones by value
                block.update(args)
                args = block.attach(sync.make_step_args(batches, dtype, stats=stats, opt=opt, step=9,
                                                        first_step=(step != 1), half_id=half_id, lr_scale=0.25))
            row = call.run(args)
            torch.cuda.synchronize()
            agg_h, rows_h = O.sync_step(hg, batches, [(0, n, b)], opt, p_h, s1_h, s2_h if adam else None, step=step,
                                        first_step=(step == 1), want_stats=stats, half_id=half_id)
            assert torch.equal(_bits(agg_d), _bits(agg_h)), (si, step)
            if stats:
                rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
                got, want = row.cpu()[:4 + K], rows_h[0][:4 + K]
                scale = want[1:3].abs().max().clamp_min(1e-300)
                assert bool(((got - want).abs() <= rtol * want.abs() + 1e-9 * scale).all()), (si, step)
            else:
                assert row is None
            if opt:
                assert torch.equal(_bits(p_d), _bits(p_h)), (si, step)
                assert torch.equal(_bits(s1_d), _bits(s1_h)), (si, step)
                if adam:
                    assert torch.equal(_bits(s2_d), _bits(s2_h)), (si, step)


def test_plan_with_nothing_but_empty_spans(gpu):
    """No workgroup to launch: the statistics rows still come back, all zero, and nothing is touched."""
    from jabas_amd import sync, _lib as L
    g = [torch.zeros(16, device=gpu) for _ in range(2)]
    p, m = torch.ones(16, device=gpu), torch.zeros(16, device=gpu)
    spans = [sync.SpanSpec([t[4:4] for t in g], agg_out=g[0][4:4], param=p[4:4], state1=m[4:4]) for _ in range(3)]
    plan = sync.SyncPlan(spans, L.OPT_SGD)
    assert plan.n_chunks == 0 and plan.n_chunks_stats == 0
    rows = plan.run(sync.make_step_args((1, 1), torch.float32, stats=True, opt=SGD, step=1, first_step=True))
    torch.cuda.synchronize()
    assert rows.shape == (3, L.STATS_STRIDE) and torch.count_nonzero(rows) == 0
    assert plan.run(sync.make_step_args((1, 1), torch.float32, stats=False, opt=SGD, step=2)) is None
    torch.cuda.synchronize()
    assert torch.equal(p, torch.ones(16, device=gpu)) and torch.count_nonzero(m) == 0
