"""Three properties of the C ABI that its callers rely on:

  * it is re-entrant: comm hooks of several replicas call it from different host threads on
    different streams at the same time (reference: one thread and one stream per VSW,
    jabas/train/trainer.py:494,514,584-588). Concurrent calls on unrelated buffers must each give
    the oracle's bits;
  * it only launches kernels (no allocation, no memset, no synchronisation), so a step can be
    captured in a HIP graph and replayed. Each replay is checked against the oracle, with eager work
    and synchronisations between the replays;
  * a status it returns is the status of its own launch: a HIP error an earlier call of the thread
    left unread is neither reported as a launch failure nor cleared.
"""
import threading

import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

SGD = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
           groups=[dict(lr=0.1, weight_decay=0.0), dict(lr=0.1, weight_decay=1e-4)])
ADAMW = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
             groups=[dict(lr=5e-4, weight_decay=0.0), dict(lr=5e-4, weight_decay=0.05)])
ADAM = dict(kind="adam", betas=(0.9, 0.999), eps=1e-8, groups=[dict(lr=2e-3, weight_decay=0.0),
                                                                dict(lr=2e-3, weight_decay=1e-2)])


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int32)


def _grads(K, n, seed, dtype=torch.float32):
    return [(torch.randn(n, generator=torch.Generator().manual_seed(9000 + 31 * seed + k)) * 1e-3).to(dtype)
            for k in range(K)]


def test_concurrent_calls_from_host_threads_on_separate_streams(gpu):
    from jabas_amd import sync
    cases = [  # K, batches, dtype, opt, n
        (2, (32, 32), torch.float32, SGD, 700001),
        (4, (48, 32, 32, 16), torch.float32, ADAMW, 500003),
        (3, (4, 2, 2), torch.float32, ADAM, 300007),
        (8, tuple(range(64, 0, -8)), torch.bfloat16, ADAMW, 400001),
        (5, (5, 4, 3, 2, 1), torch.bfloat16, SGD, 600011),
        (1, (32,), torch.float32, ADAM, 200003),
    ]
    steps = 6
    work, errors = [], []
    for i, (K, batches, dtype, opt, n) in enumerate(cases):
        hg = _grads(K, n, i, dtype)
        p_h = torch.randn(n, generator=torch.Generator().manual_seed(50 + i)) * 0.05
        adam = opt["kind"] != "sgd"
        d = dict(K=K, batches=batches, dtype=dtype, opt=opt, n=n, adam=adam, hg=hg, p_h=p_h,
                 s1_h=torch.zeros(n), s2_h=torch.zeros(n), bounds=((0, 1), (n // 3, 0), (n // 3 + 5, 1)),
                 dg=[t.to(gpu) for t in hg], agg=torch.zeros(n, device=gpu), p=p_h.to(gpu),
                 s1=torch.zeros(n, device=gpu), s2=torch.zeros(n, device=gpu),
                 ws=sync.Workspace.for_span(n, dtype, gpu), stream=torch.cuda.Stream(gpu), rows=[])
        d["span"] = sync.SpanSpec(d["dg"], agg_out=d["agg"], param=d["p"], state1=d["s1"],
                                  state2=d["s2"] if adam else None, bounds=d["bounds"])
        work.append(d)
    torch.cuda.synchronize()
    start = threading.Barrier(len(work))

    def worker(d):
        try:
            start.wait()
            with torch.cuda.stream(d["stream"]):
                for step in range(1, steps + 1):
                    args = sync.make_step_args(d["batches"], d["dtype"], stats=True, opt=d["opt"], step=step,
                                               first_step=(step == 1))
                    row = sync.sync_bucket(d["span"], args, workspace=d["ws"])
                    d["rows"].append(row.clone())            # on this thread's stream, after the step
        except Exception as exc:                             # surfaced in the main thread
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(d,)) for d in work]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i, d in enumerate(work):
        for step in range(1, steps + 1):
            agg_h, rows_h = O.sync_step(d["hg"], d["batches"], [(0, d["n"], d["bounds"])], d["opt"], d["p_h"],
                                        d["s1_h"], d["s2_h"] if d["adam"] else None, step=step,
                                        first_step=(step == 1), want_stats=True)
            rtol = 1e-2 if d["dtype"] == torch.bfloat16 else 1e-6
            got, want = d["rows"][step - 1].cpu()[:4 + d["K"]], rows_h[0][:4 + d["K"]]
            assert torch.allclose(got, want, rtol=rtol, atol=1e-30), (i, step)
        assert torch.equal(_bits(d["agg"]), _bits(agg_h)), i
        assert torch.equal(_bits(d["p"]), _bits(d["p_h"])), i
        assert torch.equal(_bits(d["s1"]), _bits(d["s1_h"])), i
        if d["adam"]:
            assert torch.equal(_bits(d["s2"]), _bits(d["s2_h"])), i


def test_fused_step_replays_in_a_hip_graph(gpu):
    """SGD-momentum step (every scalar of the launch is constant from step 2 on) over a ragged
    three-span plan with statistics, aggregated in place into VSW 0's buffers."""
    from jabas_amd import sync, _lib as L
    K, batches = 3, (4, 2, 2)
    sizes, gaps = [5000, 250001, 1], [0, 3, 1]
    offs, off = [], 0
    for s, gp in zip(sizes, gaps):
        off += gp
        offs.append(off)
        off += s
    total = off
    fresh = [_grads(K, total, 100 + r) for r in range(5)]            # one gradient set per step
    p_h = torch.randn(total, generator=torch.Generator().manual_seed(3)) * 0.05
    buf_h = torch.zeros(total)
    dg = [torch.zeros(total, device=gpu) for _ in range(K)]
    p_d, buf_d = p_h.to(gpu), torch.zeros(total, device=gpu)
    spans_h, spans_d = [], []
    for o, s in zip(offs, sizes):
        bounds = ((0, 0), (s // 2, 1)) if s > 1 else ((0, 1),)
        spans_h.append((o, s, bounds))
        sl = slice(o, o + s)
        spans_d.append(sync.SpanSpec([g[sl] for g in dg], agg_out=dg[0][sl], param=p_d[sl], state1=buf_d[sl],
                                     bounds=bounds))
    plan = sync.SyncPlan(spans_d, L.OPT_SGD)

    def load(r):
        for k in range(K):
            dg[k].copy_(fresh[r][k])

    def check(r, step, rows):
        agg_h, rows_h = O.sync_step([t.clone() for t in fresh[r]], batches, spans_h, SGD, p_h, buf_h, None,
                                    step=step, first_step=(step == 1), want_stats=True)
        for o, s, _ in spans_h:
            assert torch.equal(_bits(dg[0][o:o + s]), _bits(agg_h[o:o + s])), (r, step)
        assert torch.allclose(rows.cpu()[:, :4 + K], rows_h[:, :4 + K], rtol=1e-6, atol=1e-30), (r, step)
        assert torch.equal(_bits(p_d), _bits(p_h)), (r, step)
        assert torch.equal(_bits(buf_d), _bits(buf_h)), (r, step)

    # step 1 eagerly (first_step is a launch scalar: the momentum buffer is written, not read)
    load(0)
    rows = plan.run(sync.make_step_args(batches, torch.float32, stats=True, opt=SGD, step=1, first_step=True))
    torch.cuda.synchronize()
    check(0, 1, rows)

    # capture step >= 2
    args = sync.make_step_args(batches, torch.float32, stats=True, opt=SGD, step=2, first_step=False)
    side = torch.cuda.Stream(gpu)
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    load(1)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        plan.run(args)                                               # warm-up on the capture stream
    torch.cuda.synchronize()
    check(1, 2, plan.ws.stats)
    with torch.cuda.graph(graph, stream=side):
        plan.run(args)
    torch.cuda.synchronize()
    for r, step in ((2, 3), (3, 4), (4, 5)):
        load(r)                                                      # eager work between replays
        scratch = (dg[1] * 2.0).sum()                                # a library reduction too
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(scratch)
        check(r, step, plan.ws.stats)


def test_a_stale_hip_error_of_the_calling_thread_is_not_reported_as_ours(gpu):
    """An earlier, unrelated HIP call of the thread failed and nobody read its status. The library's
    launch must report its own status (OK), and leave that stale status where it was."""
    import ctypes as C
    from jabas_amd import _lib as L
    hip = C.CDLL("libamdhip64.so")
    hip.hipFree.argtypes, hip.hipFree.restype = [C.c_void_p], C.c_int
    hip.hipGetLastError.restype = C.c_int
    n = 100000
    g = [torch.randn(n, device=gpu) for _ in range(2)]
    out = torch.empty(n, device=gpu)
    want = O.aggregate([t.cpu() for t in g], (3, 1))
    ptrs = (C.c_void_p * 2)(g[0].data_ptr(), g[1].data_ptr())
    w = (C.c_float * 2)(*[float(x) for x in O.batch_weights((3, 1))[0]])
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    lib = L.lib()
    assert hip.hipFree(C.c_void_p(0x10)) != 0                    # fails, leaves its status in the thread's last-error slot
    rc = lib.jabas_aggregate(ptrs, 2, L.F32, w, out.data_ptr(), n, stream)
    stale = hip.hipGetLastError()                                # read (and clear) it before torch sees it
    assert rc == L.OK
    assert stale != 0, "the library swallowed the caller's pending HIP status"
    assert hip.hipGetLastError() == 0
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().view(torch.int32), want.view(torch.int32))
