"""The entry point that allocates nothing, ``jabas_sync_bucket_static``, through the C ABI: against the CPU
oracle (aggregate, weights and optimizer state bit for bit, statistics within their bar) and against
``jabas_sync_bucket`` (everything bit for bit, the statistics row included), on two calls in a row, the second
over a smaller span (the static scratch still holds the first call's partial rows). Collected last: a failure
here must not hide other tests."""
import ctypes as C

import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _oracle(n, K, seed, dtype, kind, step):
    """The same call on the host: (aggregate, weights, state1, state2, statistics row)."""
    grads, p, m, v = _case("cpu", n, K, seed, dtype, kind)
    bounds = ((0, 1), (n // 3, 0)) if n >= 3 else ()
    opt = dict(kind=kind, betas=(0.9, 0.999), eps=1e-8, momentum=0.9,
               groups=[dict(lr=5e-4, weight_decay=0.05), dict(lr=5e-4, weight_decay=0.0)])
    agg, rows = O.sync_step(grads, tuple(range(K, 0, -1)), [(0, n, bounds)], opt, p, m, v if kind != "sgd" else None,
                            step=step, first_step=False, want_stats=True)
    return agg, p, m, v, rows[0]


def _case(gpu, n, K, seed, dtype, opt_kind):
    gen = torch.Generator().manual_seed(seed)
    grads = [(torch.randn(n, generator=gen) * 1e-3).to(dtype).to(gpu) for _ in range(K)]
    p = (torch.randn(n, generator=gen) * 0.05).to(gpu)
    m = (torch.randn(n, generator=gen) * 1e-3).to(gpu)
    v = (torch.rand(n, generator=gen) * 1e-6).to(gpu)
    return grads, p, m, v


def _run(entry, gpu, n, K, seed, dtype, kind, step):
    from jabas_amd import sync, _lib as L
    grads, p, m, v = _case(gpu, n, K, seed, dtype, kind)
    agg = grads[0] if dtype == torch.float32 else torch.empty(n, device=gpu)
    fan = torch.zeros(n, device=gpu)
    bounds = ((0, 1), (n // 3, 0)) if n >= 3 else ()
    opt = dict(kind=kind, betas=(0.9, 0.999), eps=1e-8, momentum=0.9,
               groups=[dict(lr=5e-4, weight_decay=0.05), dict(lr=5e-4, weight_decay=0.0)])
    span = sync.SpanSpec(grads, agg_out=agg, param=p, state1=m, state2=v if kind != "sgd" else None, fanout=[fan],
                         bounds=bounds)
    args = sync.make_step_args(tuple(range(K, 0, -1)), dtype, stats=True, opt=opt, step=step, first_step=False)
    bd = sync.bounds_to_device(span.bounds, gpu) if span.bounds else None
    row = torch.full((L.STATS_STRIDE,), -1.0, dtype=torch.float64, device=gpu)
    torch.cuda.synchronize()
    if entry == "static":
        before = torch.cuda.memory_stats(gpu)["allocation.all.allocated"]
        sync.sync_bucket_static(span, args, stats_out=row, bounds_dev=bd)
        assert torch.cuda.memory_stats(gpu)["allocation.all.allocated"] == before, "the call allocated through torch"
    else:
        ws = sync.Workspace.for_span(n, dtype, gpu)
        c_span = span.to_c()
        L.check(L.lib().jabas_sync_bucket(C.byref(c_span), None if bd is None else bd.data_ptr(), C.byref(args),
                                          row.data_ptr(), ws.buf.data_ptr(), ws.nbytes, sync._stream_ptr()),
                "jabas_sync_bucket")
    torch.cuda.synchronize()
    return [t.clone() for t in (agg, p, m, v, fan, row)]


@pytest.mark.parametrize("K,dtype,kind", [(4, torch.float32, "adamw"), (8, torch.bfloat16, "adamw"),
                                          (3, torch.float32, "sgd")])
def test_static_entry_matches_sync_bucket_on_two_calls_the_second_smaller(gpu, K, dtype, kind):
    for call, n in enumerate((3_000_017, 70_001)):             # 1466 partial rows, then 35
        got = _run("static", gpu, n, K, 31 + call, dtype, kind, step=2 + call)
        want = _run("plain", gpu, n, K, 31 + call, dtype, kind, step=2 + call)
        for name, a, b in zip(("aggregate", "weights", "state1", "state2", "fan-out", "statistics"), got, want):
            same = torch.equal(a.view(torch.int64) if a.dtype == torch.float64 else a.view(torch.int32),
                               b.view(torch.int64) if b.dtype == torch.float64 else b.view(torch.int32))
            assert same, (call, n, name)
        assert float(got[5][3]) > 0.0
        # and against the oracle itself, not only through the other entry point
        agg_h, p_h, m_h, v_h, row_h = _oracle(n, K, 31 + call, dtype, kind, 2 + call)
        names = ("aggregate", "weights", "state1") + (("state2",) if kind != "sgd" else ())
        for name, a, b in zip(names, got, (agg_h, p_h, m_h, v_h)):
            assert torch.equal(a.cpu().view(torch.int32), b.view(torch.int32)), (call, n, name, "oracle")
        assert torch.equal(got[4].cpu().view(torch.int32), p_h.view(torch.int32)), (call, n, "fan-out", "oracle")
        row = got[5].cpu()
        rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
        assert torch.allclose(row[1:4 + K], row_h[1:4 + K], rtol=rtol, atol=0.0), (call, n, "statistics", "oracle")
        assert abs(float(row[0] - row_h[0])) <= rtol * float(torch.sqrt(row_h[1] * row_h[2])), (call, n, "dot", "oracle")


def test_static_entry_without_statistics_and_size_limit(gpu):
    from jabas_amd import sync, _lib as L
    n = 10_000
    g = [torch.randn(n, device=gpu) for _ in range(2)]
    want = torch.add(torch.mul(g[0], 0.5), torch.mul(g[1], 0.5))
    span = sync.SpanSpec(g, agg_out=g[0])
    sync.sync_bucket_static(span, sync.make_step_args((1, 1), torch.float32))
    torch.cuda.synchronize()
    assert torch.equal(g[0], want)
    # one element beyond the limit: refused before anything is launched (the pointers are never read)
    c_span = span.to_c()
    c_span.numel = L.STATIC_MAX_NUMEL + 1
    args = sync.make_step_args((1, 1), torch.float32, stats=True)
    row = torch.zeros(L.STATS_STRIDE, dtype=torch.float64, device=gpu)
    rc = L.lib().jabas_sync_bucket_static(C.byref(c_span), None, C.byref(args), row.data_ptr(), sync._stream_ptr())
    assert rc == L.ERR_SIZE
