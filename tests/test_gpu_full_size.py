"""The five benchmark configurations at their full sizes on the GPU, checked through
size-independent properties and through the oracle on sampled windows:

  * sampled windows (8 x 64 Ki elements, incl. the first and last of the arena): aggregate
    bit-exact, weights/state within 1e-6 of the oracle after two steps;
  * power-of-two scaling of every gradient scales the aggregate exactly (linearity);
  * checksum: sum(aggregate) = sum_k w_k sum(g_k) within rounding;
  * statistics: per-bucket rows add up to the row of one whole-arena span; per-worker norms
    equal a float64 library reduction; bit-identical across two runs;
  * exact-zero gradient rows (GNMT embedding) stay +0 in the aggregate and leave Adam's
    weights untouched on the first step;
  * first Adam step is the closed-form sign step where weight decay is 0;
  * every replica's weights equal the main weights (fan-out).
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from jabas_amd import _lib as L

pytestmark = pytest.mark.gpu

WINDOW = 65536


def _fill(eng, cfg, seed):
    from jabas_amd import workloads as W
    dev = eng.device
    gen = torch.Generator(device=dev).manual_seed(seed)
    live = torch.zeros(eng.layout.total, dtype=torch.bool, device=dev)       # padding between buckets stays zero
    for off, n, _, _ in eng.layout.spans:
        live[off:off + n] = True
    for k in range(eng.K):
        t = torch.randn(eng.layout.total, generator=gen, device=dev) * cfg.grad_std
        eng.grads[k].copy_(torch.where(live, t, torch.zeros((), device=dev)).to(eng.grad_dtype))
    eng.param.copy_(torch.where(live, torch.randn(eng.layout.total, generator=gen, device=dev) * 0.05,
                                torch.zeros((), device=dev)))
    if cfg.name == "gnmt":
        i = [s.name for s in cfg.specs].index(W.GNMT_EMBEDDING)
        keep = (torch.rand(W.GNMT_EMBEDDING_ROWS, generator=torch.Generator().manual_seed(0)) < 0.1).to(dev)
        for k in range(eng.K):
            v = eng.grad_view(k, i).view(W.GNMT_EMBEDDING_ROWS, W.GNMT_EMBEDDING_COLS)
            v.copy_(torch.where(keep[:, None], v, torch.zeros((), device=dev, dtype=v.dtype)))
        return i, keep
    return None, None


def _windows(eng):
    """Windows inside spans (so the oracle sees the same group bounds)."""
    rng = np.random.RandomState(7)
    out = []
    spans = eng.layout.spans
    picks = [0, len(spans) - 1] + list(rng.randint(0, len(spans), size=6))
    for si in picks:
        off, n, bounds, _ = spans[si]
        w = min(WINDOW, n)
        start = 0 if si == 0 else (n - w if si == len(spans) - 1 else int(rng.randint(0, n - w + 1)))
        out.append((off, n, bounds, start, w))
    return out


def _window_bounds(bounds, start, w):
    """Group bounds of span-local range [start, start+w), rebased to the window."""
    b = [(0, [g for s, g in bounds if s <= start][-1])] if bounds else [(0, 0)]
    for s, g in bounds:
        if start < s < start + w:
            b.append((s - start, g))
    return tuple(b)


def _close(a, b, rtol, atol):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    return bool(((a - b).abs() <= rtol * b.abs() + atol).all())


@pytest.mark.parametrize("name", ["resnet50", "vit_b16", "faster_rcnn_r50_fpn", "gnmt", "vit_l16"])
def test_full_size_configuration(gpu, name):
    from jabas_amd import workloads as W, sync
    from jabas_amd.engine import VSWFlatSync
    cfg = W.config(name)
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    print(f"full size {name}: {sum(s.numel for s in cfg.specs)} elements K={cfg.K}", flush=True)
    eng = VSWFlatSync(cfg.specs, cfg.batches, grad_dtype=gdt, opt=cfg.opt, device=gpu, n_fanout=1)
    emb, keep = _fill(eng, cfg, 11)
    wins = _windows(eng)
    adam = cfg.opt["kind"] != "sgd"
    # host copies of the sampled windows before the step
    host = []
    for off, n, bounds, start, w in wins:
        sl = slice(off + start, off + start + w)
        host.append(dict(g=[g[sl].cpu() for g in eng.grads], p=eng.param[sl].cpu(),
                         s1=torch.zeros(w), s2=torch.zeros(w), bounds=_window_bounds(bounds, start, w)))
    g_sums = [g.double().sum().item() for g in eng.grads]
    g_abs = sum(g.double().abs().sum().item() * wk for g, wk in zip(eng.grads, O.batch_weights(cfg.batches)[0]))
    norms = [(g.double() ** 2).sum().item() for g in eng.grads]
    p0 = eng.param.clone()
    g_before = [g.clone() for g in eng.grads]

    rows = eng.step(stats=True)
    torch.cuda.synchronize()
    rows1 = rows.cpu().clone()

    # ---- sampled windows against the oracle, step 1
    for h, (off, n, bounds, start, w) in zip(host, wins):
        sl = slice(off + start, off + start + w)
        agg_h, _ = O.sync_step(h["g"], cfg.batches, [(0, w, h["bounds"])], cfg.opt, h["p"], h["s1"],
                               h["s2"] if adam else None, step=1, first_step=True)
        assert torch.equal(eng.agg[sl].cpu().view(torch.int32), agg_h.view(torch.int32)), (name, off, start)
        assert _close(eng.param[sl], h["p"], 1e-6, 1e-9)
        assert _close(eng.state1[sl], h["s1"], 1e-6, 2e-9)
        if adam:
            assert _close(eng.state2[sl], h["s2"], 1e-6, 1e-16)
        h["agg"] = agg_h

    # ---- checksum of the aggregate
    w = O.batch_weights(cfg.batches)[0]
    want_sum = sum(wk * s for wk, s in zip(w, g_sums))
    got_sum = eng.agg.double().sum().item()
    assert abs(got_sum - want_sum) <= 1e-6 * g_abs + 1e-12

    # ---- statistics
    # fp32 gradients: fp64 sums throughout; bf16 gradients: fp32 partial sums per thread and chunk (bar 1e-2)
    stat_rel = 1e-10 if cfg.grad_dtype != "bf16" else 1e-5
    whole = rows1.sum(0)
    for k in range(cfg.K):
        assert whole[4 + k].item() == pytest.approx(norms[k], rel=stat_rel)
    assert whole[3].item() == pytest.approx((eng.agg.double() ** 2).sum().item(), rel=stat_rel)
    one_span = sync.gradient_stats(g_before, cfg.batches).cpu()          # one span over the whole arena
    assert torch.allclose(whole[:4 + cfg.K], one_span[:4 + cfg.K], rtol=stat_rel / 10, atol=0.0)
    cos = sync.cosine_from_stats(rows1)
    assert -1.0 <= cos <= 1.0

    # ---- fan-out and closed forms
    assert torch.equal(eng.fanout[0], eng.param)
    if adam:
        # groups without weight decay: p1 = p0 - lr * g / (|g| + eps); AdamW scales p0 by (1 - lr*wd) elsewhere
        for off, n, bounds, _ in eng.layout.spans[:3]:
            for j, (s, grp) in enumerate(bounds):
                e = bounds[j + 1][0] if j + 1 < len(bounds) else n
                hp = cfg.opt["groups"][grp]
                if hp["weight_decay"] != 0.0:
                    continue
                sl = slice(off + s, off + e)
                g = eng.agg[sl].double()
                want = p0[sl].double() - hp["lr"] * g / (g.abs() + 1e-8)
                assert torch.allclose(eng.param[sl].double(), want, rtol=2e-6, atol=1e-9)
    if emb is not None:
        rows_, cols_ = keep.numel(), W.GNMT_EMBEDDING_COLS
        a = eng.agg_view(emb).view(rows_, cols_)
        assert torch.all(a[~keep].view(torch.int32) == 0)                # exact +0 rows
        pv, p0v = eng.param_view(emb).view(rows_, cols_), eng._view(p0, emb).view(rows_, cols_)
        assert torch.equal(pv[~keep], p0v[~keep])                        # zero gradient, zero moments: no update
        assert torch.count_nonzero(eng._view(eng.state1, emb).view(rows_, cols_)[~keep]) == 0

    # ---- second step on the sampled windows (moments now non-zero)
    if gdt == torch.float32:
        for h, (off, n, bounds, start, w_) in zip(host, wins):
            h["g"][0] = h["agg"].clone()                                 # in place: VSW 0's bucket holds the aggregate
    eng.step(stats=False)
    torch.cuda.synchronize()
    for h, (off, n, bounds, start, w_) in zip(host, wins):
        sl = slice(off + start, off + start + w_)
        agg_h, _ = O.sync_step(h["g"], cfg.batches, [(0, w_, h["bounds"])], cfg.opt, h["p"], h["s1"],
                               h["s2"] if adam else None, step=2, first_step=False)
        assert torch.equal(eng.agg[sl].cpu().view(torch.int32), agg_h.view(torch.int32))
        assert _close(eng.param[sl], h["p"], 1e-6, 1e-9)
        assert _close(eng.state1[sl], h["s1"], 1e-6, 2e-9)

    # ---- linearity under power-of-two scaling and run-to-run determinism, on fresh engines
    del eng
    torch.cuda.empty_cache()
    a = VSWFlatSync(cfg.specs, cfg.batches, grad_dtype=gdt, opt=None, device=gpu, in_place=False)
    for k in range(cfg.K):
        a.grads[k].copy_(g_before[k])
    r1 = a.step(stats=True).cpu().clone()
    agg1 = a.agg.clone()
    r2 = a.step(stats=True).cpu().clone()
    assert torch.equal(r1.view(torch.int64), r2.view(torch.int64))       # same plan, same bits
    if cfg.K <= L.STATS_GRAM_MAX_K:
        # the worker x worker products out of the same launch: the row's other slots keep their bits; the pair sums
        # equal a float64 library reduction; and the sums of the halves and of the aggregate are the quadratic
        # forms of the Gram matrix in the weights (up to the fp32 rounding of the aggregated elements)
        K = cfg.K
        r3 = a.step(stats="gram").cpu().clone()
        assert torch.equal(r3[:, :4 + K].view(torch.int64), r1[:, :4 + K].view(torch.int64))
        G = a.gram(r3).cpu()
        for i in range(K):
            for j in range(i + 1, K):
                want = (a.grads[i].double() * a.grads[j].double()).sum().item()
                assert abs(G[i, j].item() - want) <= stat_rel * (norms[i] * norms[j]) ** 0.5
        wv, half, whv = O.batch_weights(cfg.batches)
        wv = torch.tensor(wv, dtype=torch.float64)
        wa = torch.tensor([x if h == 0 else 0.0 for x, h in zip(whv, half)], dtype=torch.float64)
        wb = torch.tensor([x if h == 1 else 0.0 for x, h in zip(whv, half)], dtype=torch.float64)
        tot = r3.sum(0)
        assert float(wv @ G @ wv) == pytest.approx(tot[3].item(), rel=1e-5)
        assert float(wa @ G @ wa) == pytest.approx(tot[1].item(), rel=1e-5)
        if K > 1:
            assert float(wb @ G @ wb) == pytest.approx(tot[2].item(), rel=1e-5)
            assert abs(float(wa @ G @ wb) - tot[0].item()) <= 1e-5 * (tot[1].item() * tot[2].item()) ** 0.5
    for k in range(cfg.K):
        a.grads[k].mul_(4.0)
    a.step(stats=False)
    torch.cuda.synchronize()
    assert torch.equal((agg1 * 4.0).view(torch.int32), a.agg.view(torch.int32))


def test_gnmt_embedding_rows_with_independent_masks(gpu):
    """The GNMT embedding bucket (32,317 x 1,024) at full size where every VSW saw its own 10 % of
    the rows: a row of the aggregate is exactly +0 only where no VSW touched it, Adam's first
    step leaves exactly those weights alone, and the whole aggregate is bit-exact."""
    from jabas_amd import workloads as W, sync
    cfg = W.config("gnmt")
    rows, cols = W.GNMT_EMBEDDING_ROWS, W.GNMT_EMBEDDING_COLS
    n, K = rows * cols, cfg.K
    hg, keeps = [], []
    for k in range(K):
        gen = torch.Generator().manual_seed(4321 + k)
        keep = torch.rand(rows, generator=gen) < 0.1
        g = (torch.randn(rows, cols, generator=gen) * cfg.grad_std) * keep[:, None]
        hg.append(torch.where(keep[:, None], g, torch.zeros(())).reshape(-1).contiguous())
        keeps.append(keep)
    touched = torch.stack(keeps).any(0)
    assert 0.3 < touched.float().mean() < 0.4                               # 1 - 0.9^4 = 0.344
    p_h = torch.randn(n, generator=torch.Generator().manual_seed(9)) * 0.05
    p0 = p_h.clone()
    m_h, v_h = torch.zeros(n), torch.zeros(n)
    dg = [t.to(gpu) for t in hg]
    p_d, m_d, v_d = p_h.to(gpu), torch.zeros(n, device=gpu), torch.zeros(n, device=gpu)
    span = sync.SpanSpec(dg, agg_out=dg[0], param=p_d, state1=m_d, state2=v_d)
    args = sync.make_step_args(cfg.batches, torch.float32, stats=True, opt=cfg.opt, step=1, first_step=True)
    row = sync.sync_bucket(span, args)
    torch.cuda.synchronize()
    agg_h, rows_h = O.sync_step(hg, cfg.batches, [(0, n, ((0, 0),))], cfg.opt, p_h, m_h, v_h, step=1,
                                first_step=True, want_stats=True)
    agg_d = dg[0].cpu()
    assert torch.equal(agg_d.view(torch.int32), agg_h.view(torch.int32))
    a2 = agg_d.view(rows, cols)
    assert torch.all(a2[~touched].view(torch.int32) == 0)                   # +0, not -0
    assert torch.all((a2[touched] != 0).any(1))
    p2 = p_d.cpu().view(rows, cols)
    assert torch.equal(p2[~touched], p0.view(rows, cols)[~touched])
    assert torch.equal(p_d.cpu().view(torch.int32), p_h.view(torch.int32))
    assert torch.equal(m_d.cpu().view(torch.int32), m_h.view(torch.int32))
    assert torch.equal(v_d.cpu().view(torch.int32), v_h.view(torch.int32))
    assert torch.allclose(row.cpu()[:4 + K], rows_h[0][:4 + K], rtol=1e-6, atol=0.0)
    for k in range(K):                                                      # per-worker norms: only that worker's rows count
        assert row[4 + k].item() == pytest.approx((hg[k].double() ** 2).sum().item(), rel=1e-10)


@pytest.mark.parametrize("K", [8, 13])
def test_gram_bf16_long_span(gpu, K):
    """bf16 Gram over a span long enough (2^28 + 77 elements) that every wave moves its fp32 running sums
    into the fp64 sums several times before the last one. The K workers point at three distinct buffers
    (the kernel only reads), so every entry is one of six dot products, which a float64 library reduction gives."""
    from jabas_amd import sync
    n = (1 << 28) + 77
    gen = torch.Generator(device=gpu).manual_seed(99)
    bufs = [(torch.randn(n + 8, generator=gen, device=gpu) * 1e-2).to(torch.bfloat16) for _ in range(3)]
    views = [b[s:s + n] for b, s in zip(bufs, (0, 4, 0))]
    which = [(k * 7 + k // 3) % 3 for k in range(K)]
    G = sync.gram([views[w] for w in which]).cpu()
    dots = torch.zeros(3, 3, dtype=torch.float64)
    for a in range(3):
        for b in range(a, 3):
            s = 0.0
            for c in range(0, n, 1 << 26):                                  # chunks: bounded float64 temporaries
                s += (views[a][c:c + (1 << 26)].double() * views[b][c:c + (1 << 26)].double()).sum().item()
            dots[a, b] = dots[b, a] = s
    for a in range(K):
        for b in range(K):
            scale = (dots[which[a], which[a]] * dots[which[b], which[b]]).sqrt().item()
            assert abs(G[a, b].item() - dots[which[a], which[b]].item()) <= 5e-6 * scale, (a, b)
    assert torch.equal(G, G.t())
