#!/usr/bin/env python3
"""Benchmark of the fused per-GPU gradient-sync step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-all] [--no-cpu] [--no-extras]
                    [--cpu-seconds S] [--calibrate-copy] [--flat-moments]

A step is one fused sync step (batch-weighted aggregate of the K VSW gradient buckets
+ the similarity statistics where the configuration asks for them + optimizer update) over
one full synthetic gradient set. The headline workload is the largest configuration that
fits one GPU, ViT-L/16 (304 M parameters, K = 8 bf16 gradient sets, AdamW); the other four
configurations are timed too and reported under "workloads" in the same JSON line. Inputs
are resident in HBM before the timed region starts. Small configurations rotate over
several copies of their buffers so that the working set stays far above the 256 MB
last-level cache.

Prints ONE JSON line: metric sync_step_GBps = algorithmic bytes per step / time per step,
with a "roofline" object (HBM-bound; achieved = algorithmic bytes per launch / mean launch
duration = HIP-event time of the timed region on the launching stream / its launches) and a
"cpu_baseline" object (the reference's unfused PyTorch structure timed on this box's host
cores, rank 0 only, a bounded number of whole steps). Every entry of "workloads" carries
its own figures of both, the step as the reference's calling convention reaches it (one
hook call per bucket and VSW: one launch per bucket, per 64 MiB of buckets, per step), and the neighbouring launches
(without statistics, with full statistics rows).
"""
import argparse
import gc
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published peak
ROTATE_TARGET_BYTES = 1.5e9   # minimum total working set per configuration
TRAFFIC_FILE = os.path.join("profiles", "fused_kernel_hbm_traffic.json")


def measured_traffic(name):
    """HBM bytes per launch of the fused kernel from rocprofv3 counters, read from the tracked summary
    next to the profile it came from (None when that file does not cover the workload)."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            table = json.load(f)
        return table["workloads"].get(name, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError, KeyError):
        return None


def algorithmic_bytes_per_elem(cfg):
    s_g = 2 if cfg.grad_dtype == "bf16" else 4
    state = 16 if cfg.opt["kind"] == "sgd" else 24
    return cfg.K * s_g + 4 + state


def fill_engine(eng, cfg, device, torch, seed, independent_masks=False):
    from jabas_amd import workloads as W
    gdt = eng.grad_dtype
    gen = torch.Generator(device=device).manual_seed(seed)
    for k in range(cfg.K):
        tmp = torch.randn(eng.layout.total, generator=gen, device=device, dtype=torch.float32) * cfg.grad_std
        eng.grads[k].copy_(tmp.to(gdt))
        del tmp
    eng.param.copy_(torch.randn(eng.layout.total, generator=gen, device=device) * 0.05)
    if cfg.name == "gnmt":
        # embedding gradient: a fixed random 10 % of the rows non-zero; the same rows for every VSW, or
        # (second variant) rows drawn independently per VSW
        i = [s.name for s in cfg.specs].index(W.GNMT_EMBEDDING)
        rows, cols = W.GNMT_EMBEDDING_ROWS, W.GNMT_EMBEDDING_COLS
        for k in range(cfg.K):
            mask_seed = k + 1 if independent_masks else 0
            keep = (torch.rand(rows, generator=torch.Generator().manual_seed(mask_seed)) < 0.1).to(device)
            v = eng.grad_view(k, i).view(rows, cols)
            v.copy_(torch.where(keep[:, None], v, torch.zeros((), device=device, dtype=v.dtype)))


FLAT_MOMENTS = False     # --flat-moments: Adam's moments in arrays of their own instead of the interleaved arena


def build_engines(cfg, device, torch, independent_masks=False, n_fanout=0, write_aggregate=True):
    from jabas_amd.engine import VSWFlatSync
    from jabas_amd.sync import MOMENT_BLOCK_LOG2
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    numel = sum(s.numel for s in cfg.specs)
    ws = numel * algorithmic_bytes_per_elem(cfg)
    copies = max(1, math.ceil(ROTATE_TARGET_BYTES / ws))
    engines = []
    for c in range(copies):
        eng = VSWFlatSync(cfg.specs, cfg.batches, grad_dtype=gdt, opt=cfg.opt, device=device, n_fanout=n_fanout,
                          write_aggregate=write_aggregate, moment_block_log2=0 if FLAT_MOMENTS else MOMENT_BLOCK_LOG2)
        fill_engine(eng, cfg, device, torch, 1234 + 17 * c, independent_masks)
        engines.append(eng)
    return engines, numel, copies


_last_host_us = 0.0


def timed_region(fn, steps, warmup, torch):
    """ms per call of fn(i) over exactly `steps` calls, HIP events on the current stream. The host time the
    calls themselves took (queueing only: measured before the closing synchronisation) is left in
    ``host_us_of_last_region()``."""
    global _last_host_us
    # The interpreter's cyclic garbage collector stays out of the timed region (as timeit keeps it out): a full
    # collection over everything torch has imported takes tens of milliseconds, and one that falls between the
    # opening event and the first launch leaves the GPU idle for that long (seen: 40 ms in a 120 ms region).
    # Collected before the warm-up, so that the GPU is busy again when the timed region starts.
    gc_was_on = gc.isenabled()
    gc.collect()
    gc.disable()
    try:
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        _last_host_us = (time.perf_counter() - t0) * 1e6 / steps
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
    finally:
        if gc_was_on:
            gc.enable()
    return max(e0.elapsed_time(e1), 1e-6) / steps, wall_ms / steps


def host_us_of_last_region():
    return _last_host_us


def rate(bytes_per_step, ms):
    gbps = bytes_per_step / 1e9 / (ms / 1e3)
    return dict(ms_per_step=ms, GBps=gbps, pct_hbm_peak=100.0 * gbps / HBM_PEAK_GBPS)


class _Bucket:
    """The part of a DDP GradBucket the hooks read."""

    def __init__(self, i, t):
        self._i, self._t = i, t

    def index(self):
        return self._i

    def buffer(self):
        return self._t


def hook_path(cfg, eng, device, steps, warmup, torch, deferred, batch_bytes=0, launch_streams=1):
    """The same step as the reference's calling convention reaches it: per bucket, VSW 0's similarity
    hook (with the optimizer bound: the overlap weight-sync mode) and K - 1 dummy hooks, each handing
    over its bucket view; one fused launch per bucket (or one per step, deferred) on a launch stream
    of its own. One host thread plays all K VSWs. Returns ms per step (HIP events around the steps)."""
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    pbs, bucket_slices = {}, []
    for b, (off, numel, bounds, _bucket) in enumerate(eng.layout.spans):
        sl = slice(off, off + numel)
        bucket_slices.append(sl)
        pbs[b] = dict(param=eng.param[sl], bounds=bounds, agg_out=None if eng.agg is eng.grads[0] else eng.agg[sl],
                      **eng.state_of_span(off, numel))
    stream = torch.cuda.Stream(device)
    local = LocalBucketSync(cfg.batches, opt=cfg.opt, param_buckets=pbs, deferred=deferred, stream=stream,
                            batch_bytes=batch_bytes, launch_streams=launch_streams)
    local.step_count = eng.step_count
    local._momentum_ready = eng.step_count > 0
    state = H.GradientSimilarityState(None, cfg.K + cfg.K % 2, None, [], 1 if cfg.stats else 10 ** 9).attach_local(local)
    main_hook = H.similimarity_allreduce_hook(H.subgroup_allreduce_hook)
    peers = [H.VSWPeerState(local, k) for k in range(1, cfg.K)]
    buckets = [[_Bucket(b, eng.grads[k][sl]) for k in range(cfg.K)] for b, sl in enumerate(bucket_slices)]
    cur = torch.cuda.current_stream(device)

    def one_step(_):
        for per_vsw in buckets:
            main_hook(state, per_vsw[0])
            for k in range(1, cfg.K):
                H.dummy_hook(peers[k - 1], per_vsw[k])
        local.finish_step((cur,))
        state.grad_placeholder.clear()

    for i in range(warmup):                         # the first steps create streams' and events' pools
        one_step(i)
    launched_before = local.launched
    # three timed regions: these legs are bound by the host thread, whose pace moves from run to run and box to box
    runs = sorted(timed_region(one_step, steps, 0, torch) for _ in range(3))
    ms, wall = runs[1]
    eng.step_count = local.step_count
    return dict(ms_per_step=ms, ms_per_step_min=runs[0][0], ms_per_step_max=runs[2][0], wall_ms_per_step=wall,
                launches_per_step=(local.launched - launched_before) / (3 * steps),
                host_us_per_hook_call=1e3 * wall / (cfg.K * len(buckets)), launch_streams=launch_streams)


def bucket_launches(cfg, eng, device, steps, warmup, torch, launch_streams):
    """One jabas_sync_bucket launch per bucket of the gradient set (what the per-bucket hook mode queues), with no
    hand-over events in between, bucket i on launch stream i mod launch_streams: what the GPU needs for the
    launches themselves. ms per step, HIP events on the current stream around the steps (which waits for the
    launch streams at the end of every step)."""
    from jabas_amd import sync
    calls = []
    for b, (off, numel, bounds, _bucket) in enumerate(eng.layout.spans):
        sl = slice(off, off + numel)
        calls.append(sync.BucketCall(sync.SpanSpec(
            [g[sl] for g in eng.grads], agg_out=eng.agg[sl], param=eng.param[sl], bounds=bounds,
            **eng.state_of_span(off, numel))))
    streams = [torch.cuda.Stream(device) for _ in range(launch_streams)]
    cur = torch.cuda.current_stream(device)
    level = "similarity" if cfg.stats else False

    def one_step(_):
        args = eng.step_args(stats=level)
        for s in streams:
            s.wait_stream(cur)
        for b, call in enumerate(calls):
            call.run(args, stream=streams[b % launch_streams])
        for s in streams:
            cur.wait_stream(s)
        eng.step_count += 1

    return timed_region(one_step, steps, warmup, torch)[0]


_sleep_cycles_per_us = None


def sleep_cycles_per_us(torch):
    """Cycles of torch.cuda._sleep per microsecond on this box (one wave spinning on the clock: a stand-in
    for backward work that takes time on a stream without touching HBM)."""
    global _sleep_cycles_per_us
    if _sleep_cycles_per_us is None:
        torch.cuda._sleep(1000)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = 2_000_000
        a.record()
        torch.cuda._sleep(n)
        b.record()
        torch.cuda.synchronize()
        _sleep_cycles_per_us = n / (a.elapsed_time(b) * 1e3)
    return _sleep_cycles_per_us


def hook_path_threads(cfg, eng, device, steps, warmup, torch, launch_streams, backward_factor=3.0, engine_ms=None):
    """The hook path as training runs it (jabas/train/trainer.py:327-337, 452-468, 494-514): K host threads on K
    streams, one per VSW; ahead of every bucket each VSW's stream carries a stand-in for the backward work
    that produces the bucket (a one-wave spin of backward_factor x the bucket's share of the engine step, so
    the K backward passes of a step take backward_factor x the sync step and leave HBM to the sync launches),
    then the VSW's hook is called: VSW 0's similarity hook with the optimizer bound, dummy_hook on the others.
    One fused launch per bucket, alternating between `launch_streams` launch streams.
    Reported: ms per step (HIP events from the release of the VSW streams to the end of finish_step),
    exposed_sync_ms = end of step - the moment the last VSW's stream passed its last hand-over (what the sync
    adds to a step after backward is over), host_us_per_hook_call (wall time inside the hook calls, per call,
    measured in the calling threads: includes waiting for the interpreter lock)."""
    import threading
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    K = cfg.K
    pbs, bucket_slices = {}, []
    for b, (off, numel, bounds, _bucket) in enumerate(eng.layout.spans):
        sl = slice(off, off + numel)
        bucket_slices.append(sl)
        pbs[b] = dict(param=eng.param[sl], bounds=bounds, agg_out=None if eng.agg is eng.grads[0] else eng.agg[sl],
                      **eng.state_of_span(off, numel))
    # launch_streams = 0: no launch stream, a bucket's launch on the stream of the VSW that handed it over last
    local = LocalBucketSync(cfg.batches, opt=cfg.opt, param_buckets=pbs,
                            stream=torch.cuda.Stream(device) if launch_streams else None,
                            launch_streams=launch_streams, launch_on_last_vsw=not launch_streams)
    local.step_count = eng.step_count
    local._momentum_ready = eng.step_count > 0
    state = H.GradientSimilarityState(None, K + K % 2, None, [], 1 if cfg.stats else 10 ** 9).attach_local(local)
    main_hook = H.similimarity_allreduce_hook(H.subgroup_allreduce_hook)
    peers = [None] + [H.VSWPeerState(local, k) for k in range(1, K)]
    buckets = [[_Bucket(b, eng.grads[k][sl]) for k in range(K)] for b, sl in enumerate(bucket_slices)]
    total = sum(sl.stop - sl.start for sl in bucket_slices)
    per_us = sleep_cycles_per_us(torch)
    spin = [int(backward_factor * engine_ms * 1e3 * (sl.stop - sl.start) / total * per_us) for sl in bucket_slices]
    streams = [torch.cuda.Stream(device) for _ in range(K)]
    cur = torch.cuda.current_stream(device)
    n_iter = warmup + steps
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_iter)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_iter)]
    lasts = [[torch.cuda.Event(enable_timing=True) for _ in range(K)] for _ in range(n_iter)]
    go, done = threading.Barrier(K + 1), threading.Barrier(K + 1)
    host_s, errors = [0.0] * K, []

    def vsw(k):
        torch.cuda.set_device(device)
        hook, st = (main_hook, state) if k == 0 else (H.dummy_hook, peers[k])
        try:
            with torch.cuda.stream(streams[k]):
                for it in range(n_iter):
                    go.wait()
                    streams[k].wait_event(starts[it])
                    spent = 0.0
                    for b, per_vsw in enumerate(buckets):
                        torch.cuda._sleep(spin[b])
                        t0 = time.perf_counter()
                        hook(st, per_vsw[k])
                        spent += time.perf_counter() - t0
                    lasts[it][k].record(streams[k])
                    if it >= warmup:
                        host_s[k] += spent
                    done.wait()
        except Exception as exc:                    # pragma: no cover - reported below
            errors.append(exc)
            go.abort()
            done.abort()

    threads = [threading.Thread(target=vsw, args=(k,), daemon=True) for k in range(K)]
    for t in threads:
        t.start()
    wall0 = 0.0
    gc_was_on = gc.isenabled()            # as in timed_region: no collection pause inside a measured step
    gc.collect()
    gc.disable()
    try:
        for it in range(n_iter):
            if it == warmup:
                torch.cuda.synchronize()
                wall0 = time.perf_counter()
            starts[it].record(cur)
            go.wait(timeout=120)
            done.wait(timeout=120)
            local.finish_step((cur,))
            ends[it].record(cur)
            state.grad_placeholder.clear()
    except threading.BrokenBarrierError:
        raise RuntimeError(f"hook threads failed: {errors}")
    finally:
        if gc_was_on:
            gc.enable()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall0) * 1e3 / steps
    for t in threads:
        t.join(timeout=30)
    ms = [starts[it].elapsed_time(ends[it]) for it in range(warmup, n_iter)]
    exposed = [min(lasts[it][k].elapsed_time(ends[it]) for k in range(K)) for it in range(warmup, n_iter)]
    backward = [max(starts[it].elapsed_time(lasts[it][k]) for k in range(K)) for it in range(warmup, n_iter)]
    eng.step_count = local.step_count
    calls = steps * K * len(buckets)
    return dict(ms_per_step=sum(ms) / len(ms), exposed_sync_ms=sum(exposed) / len(exposed),
                exposed_sync_ms_max=max(exposed), backward_stand_in_ms=sum(backward) / len(backward),
                wall_ms_per_step=wall_ms, host_us_per_hook_call=1e6 * sum(host_s) / calls,
                hook_calls_per_step=K * len(buckets), launch_streams=launch_streams,
                backward_factor=backward_factor, native_launches=local.native_launches)


def time_config(cfg, device, steps, warmup, torch, extras=True):
    engines, numel, copies = build_engines(cfg, device, torch)
    bytes_per_step = numel * algorithmic_bytes_per_elem(cfg)
    n = len(engines)
    level = "similarity" if cfg.stats else False
    # timed region: exactly `steps` steps, back to back on one stream
    ms_per_step, wall_ms = timed_region(lambda i: engines[i % n].step(stats=level), steps, warmup, torch)
    host_us_direct = host_us_of_last_region()
    # per-launch durations (instrumentation pass, outside the timed region): one event pair per step
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i, (a, b) in enumerate(evs):
        a.record()
        engines[i % n].step(stats=level)
        b.record()
    torch.cuda.synchronize()
    launch_ms = sorted(a.elapsed_time(b) for a, b in evs)
    res = dict(
        workload=cfg.name, elements=numel, K=cfg.K, batches=list(cfg.batches), grad_dtype=cfg.grad_dtype,
        optimizer=cfg.opt["kind"], stats="similarity" if cfg.stats else "none", spans=engines[0].plan.n_span,
        bytes_per_elem=algorithmic_bytes_per_elem(cfg), GB_per_step=bytes_per_step / 1e9,
        wall_ms_per_step=wall_ms, host_us_per_step=host_us_direct, buffer_copies=copies,
        launch_ms_mean=sum(launch_ms) / len(launch_ms), launch_ms_median=launch_ms[len(launch_ms) // 2],
        launch_ms_min=launch_ms[0])
    res.update(rate(bytes_per_step, ms_per_step))
    if cfg.stats and extras:
        # the step between statistic steps (statistics run every `interval` steps in training), and the
        # step that also forms the squared norm of every VSW's gradient
        ms, _ = timed_region(lambda i: engines[i % n].step(stats=False), steps, warmup, torch)
        res["step_without_statistics"] = rate(bytes_per_step, ms)
        ms, _ = timed_region(lambda i: engines[i % n].step(stats="full"), steps, warmup, torch)
        res["step_with_per_vsw_norms"] = rate(bytes_per_step, ms)
        if cfg.K <= 8:
            # the worker x worker Gram matrix ("between workers" statistics): out of the step's own launch (pair
            # products beside the full rows, no byte read twice), against the step followed by a pass of its
            # own over the K gradient arenas (K * gradient size more bytes per element read)
            from jabas_amd import sync
            ms, _ = timed_region(lambda i: engines[i % n].step(stats="gram"), steps, warmup, torch)
            res["step_with_worker_gram_in_the_launch"] = rate(bytes_per_step, ms)
            gws = torch.empty(1056 * 256, dtype=torch.float64, device=device)

            def step_then_gram(i):
                engines[i % n].step(stats="full")
                sync.gram(engines[i % n].grads, workspace=gws)
            ms, _ = timed_region(step_then_gram, steps, warmup, torch)
            res["step_then_worker_gram_pass"] = dict(ms_per_step=ms)
            del gws
    if extras:
        # the same step recorded once in a HIP graph and replayed with the scalars of the moment in a device
        # block (Adam's bias correction moves every step): one graph launch per step instead of the step's launches
        graphed = [e.capture(stats=level) for e in engines]
        ms, wall = timed_region(lambda i: graphed[i % n].replay(), steps, warmup, torch)
        # what a replay trades: the GPU pays the scalar-refresh kernel and the graph launch, the host queues one
        # graph launch (plus that refresh) instead of the step's launches
        res["recorded_step"] = dict(rate(bytes_per_step, ms), wall_ms_per_step=wall,
                                    host_us_per_step=host_us_of_last_region(), host_us_per_step_direct=host_us_direct)
        del graphed
    if extras:
        hsteps, hwarm = max(5, steps // 2), max(10, warmup)
        res["hook_path_per_bucket_ms"] = hook_path(cfg, engines[0], device, hsteps, hwarm, torch, False)
        res["hook_path_batched_64MiB_ms"] = hook_path(cfg, engines[0], device, hsteps, hwarm, torch, False, 64 << 20)
        res["hook_path_deferred_ms"] = hook_path(cfg, engines[0], device, hsteps, hwarm, torch, True)
        res["hook_path_per_bucket_2_streams_ms"] = hook_path(cfg, engines[0], device, hsteps, hwarm, torch, False,
                                                             launch_streams=2)
        # the GPU's share of the per-bucket mode: one launch per bucket, back to back, on 1, 2 and 3 launch streams
        res["bucket_launches_back_to_back_ms"] = {
            str(ls): bucket_launches(cfg, engines[0], device, hsteps, hwarm, torch, ls) for ls in (1, 2, 3)}
        # the same hooks as training calls them: K threads on K streams with backward-like work between the buckets
        # (a leg of K host threads: whatever goes wrong in it is reported in its place, not instead of the line)
        for ls in (1, 2, 0):
            key = f"hook_path_threads_{ls}_launch_stream{'s' if ls > 1 else ''}" if ls else "hook_path_threads_launch_on_last_vsw"
            try:
                res[key] = hook_path_threads(cfg, engines[0], device, hsteps, max(3, hwarm // 3), torch, ls,
                                             engine_ms=ms_per_step)
            except Exception as exc:
                torch.cuda.synchronize()
                res[key] = dict(error=f"{type(exc).__name__}: {exc}")
    if cfg.name == "gnmt" and extras:
        # global-norm clipping (examples/gnmt/seq2seq/train/trainer.py:157-161): aggregate + statistics, the
        # coefficient on the device, then the update over the scaled aggregate
        ms, _ = timed_region(lambda i: engines[i % n].step(stats=level, clip_norm=5.0), steps, warmup, torch)
        res["clipped_step_ms"] = ms
        graphed = [e.capture(stats=level, clip_norm=5.0) for e in engines]
        res["clipped_recorded_step_ms"] = timed_region(lambda i: graphed[i % n].replay(), steps, warmup, torch)[0]
        del graphed
    stats_rows = engines[0].step(stats=level) if cfg.stats else None
    res["cosine"] = engines[0].cosine(stats_rows) if stats_rows is not None else None
    res["finite"] = bool(torch.isfinite(engines[0].param).all())
    del engines
    torch.cuda.empty_cache()
    if extras and cfg.K > 1:
        # what one weight arena shared by every VSW's model saves: the same step when each of the other K - 1
        # replicas keeps weights of its own that the launch refreshes (4 (K - 1) more bytes written per element)
        engines, _, _ = build_engines(cfg, device, torch, n_fanout=cfg.K - 1)
        ms, _ = timed_region(lambda i: engines[i % len(engines)].step(stats=level), steps, warmup, torch)
        fan_bytes = numel * (algorithmic_bytes_per_elem(cfg) + 4 * (cfg.K - 1))
        res["step_with_replica_fanout"] = dict(rate(fan_bytes, ms), bytes_per_elem=fan_bytes // numel)
        del engines
        torch.cuda.empty_cache()
    if extras:
        # the step as the trainer runs it: it clears the buckets right after the update, so the launch hands the
        # aggregate to the optimizer in registers and writes it nowhere (4 bytes per element fewer)
        engines, _, _ = build_engines(cfg, device, torch, write_aggregate=False)
        ms, _ = timed_region(lambda i: engines[i % len(engines)].step(stats=level), steps, warmup, torch)
        res["trainer_step_no_aggregate_write"] = dict(rate(bytes_per_step - 4 * numel, ms),
                                                      bytes_per_elem=algorithmic_bytes_per_elem(cfg) - 4)
        del engines
        torch.cuda.empty_cache()
    if extras and cfg.opt["kind"] != "sgd":
        # the same step with amsgrad (examples/gnmt/seq2seq/train/shard_optimizer.py:58-66): the running maximum of
        # the second moment is one more state stream, 8 more bytes per element
        ams = cfg._replace(opt=dict(cfg.opt, amsgrad=True))
        engines, _, _ = build_engines(ams, device, torch)
        ms, _ = timed_region(lambda i: engines[i % len(engines)].step(stats=level), steps, warmup, torch)
        ams_bytes = numel * (algorithmic_bytes_per_elem(cfg) + 8)
        res["step_with_amsgrad"] = dict(rate(ams_bytes, ms), bytes_per_elem=ams_bytes // numel)
        del engines
        torch.cuda.empty_cache()
    if cfg.name == "gnmt" and extras:
        engines, _, _ = build_engines(cfg, device, torch, independent_masks=True)
        ms, _ = timed_region(lambda i: engines[i % len(engines)].step(stats=level), steps, warmup, torch)
        res["independent_row_masks"] = rate(bytes_per_step, ms)
        del engines
        torch.cuda.empty_cache()
    return res


def copy_rate(device, steps, torch):
    """The library's own plain copy (K = 1, weight 1 aggregate: the same 16-byte nontemporal loads and
    stores as every other instantiation) over 1 GiB: what this box's memory system gives a 1:1
    read/write stream."""
    from jabas_amd import sync
    src = torch.ones(1 << 28, dtype=torch.float32, device=device)
    dst = torch.empty_like(src)
    ms, _ = timed_region(lambda i: sync.aggregate([src], (1,), out=dst), max(5, steps // 5), 2, torch)
    del src, dst
    torch.cuda.empty_cache()
    return 2 * (1 << 30) / 1e9 / (ms / 1e3)


def device_info(device, torch):
    """What tells one box from another (boxes of the same model differ by several points on mixed read/write
    streams): the device's name and clocks as torch reports them, and the clocks and partition modes `rocm-smi`
    shows at this moment (a child process; absent tool or odd output: left out)."""
    import subprocess
    p = torch.cuda.get_device_properties(device)
    info = dict(name=p.name, compute_units=p.multi_processor_count, memory_GiB=round(p.total_memory / 2 ** 30, 1),
                gcn_arch=getattr(p, "gcnArchName", None), clock_MHz=getattr(p, "clock_rate", 0) / 1e3 or None,
                memory_clock_MHz=getattr(p, "memory_clock_rate", 0) / 1e3 or None,
                l2_MiB=round(getattr(p, "L2_cache_size", 0) / 2 ** 20, 1) or None)
    try:
        out = subprocess.run(["rocm-smi", "--showclocks", "--showmemorypartition", "--showcomputepartition", "--json"],
                             capture_output=True, text=True, timeout=20)
        cards = json.loads(out.stdout)
        card = cards.get("card0") or next(iter(cards.values()))
        info["rocm_smi"] = {k: v for k, v in card.items()
                            if any(w in k.lower() for w in ("mclk", "sclk", "fclk", "socclk", "partition"))}
    except Exception:
        pass
    return info


def statistics_launches(device, steps, torch):
    """The similarity hook on a step without weight update (the sequential weight-sync mode): aggregate +
    statistics over a 64 Mi-element bucket set, and the statistics alone, K = 4 and 8, fp32 and bf16."""
    from jabas_amd import sync
    n = 1 << 26
    out = []
    for K in (4, 8):
        for gdt, name, sg in ((torch.float32, "f32", 4), (torch.bfloat16, "bf16", 2)):
            grads = [(torch.randn(n, device=device) * 1e-3).to(gdt) for _ in range(K)]
            agg = torch.empty(n, device=device)
            batches = tuple(range(K, 0, -1))
            entry = dict(K=K, grad_dtype=name, elements=n)
            for level in ("similarity", "full"):
                args = sync.make_step_args(batches, gdt, stats=level)
                ws = sync.Workspace.for_span(n, gdt, device)
                span = sync.SpanSpec(grads, agg_out=agg)
                ms, _ = timed_region(lambda i: sync.sync_bucket(span, args, workspace=ws), max(5, steps // 2), 3, torch)
                entry[f"aggregate_and_{level}"] = rate(n * (K * sg + 4), ms)
                span = sync.SpanSpec(grads)
                ms, _ = timed_region(lambda i: sync.sync_bucket(span, args, workspace=ws), max(5, steps // 2), 3, torch)
                entry[f"{level}_only"] = rate(n * K * sg, ms)
            out.append(entry)
            del grads, agg
            torch.cuda.empty_cache()
    return out


def gram_launches(device, steps, torch):
    """The worker x worker Gram matrix ("between workers" statistics; both launches, Gram and finalize)
    over 64 Mi elements: bytes read = K x element size per element."""
    from jabas_amd import sync
    n = 1 << 26
    out = []
    for gdt, name, sg in ((torch.float32, "f32", 4), (torch.bfloat16, "bf16", 2)):
        grads = [(torch.randn(n, device=device) * 1e-3).to(gdt) for _ in range(16)]
        for K in (4, 8, 12, 16):
            ms, _ = timed_region(lambda i: sync.gram(grads[:K]), max(5, steps // 2), 3, torch)
            out.append(dict(K=K, grad_dtype=name, elements=n, **rate(n * K * sg, ms)))
        del grads
        torch.cuda.empty_cache()
    return out


def launch_modes(cfg, device, steps, torch):
    """Small-span launch overhead (the Faster R-CNN configuration's point): the same step as
    one launch over bucket spans, one launch over one span per tensor, one launch per
    bucket, and one launch per tensor. ms per step from HIP events."""
    from jabas_amd.engine import VSWFlatSync
    from jabas_amd.sync import SyncPlan
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    out = {}
    for label, per_tensor in (("one_launch_bucket_spans", False), ("one_launch_tensor_spans", True)):
        eng = VSWFlatSync(cfg.specs, cfg.batches, grad_dtype=gdt, opt=cfg.opt, device=device, per_tensor_spans=per_tensor)
        for g in eng.grads:
            g.normal_(0, cfg.grad_std)
        eng.param.normal_(0, 0.05)
        eng.step()
        out[label] = dict(launches=1, spans=eng.plan.n_span, ms=timed_region(lambda i: eng.step(), steps, 3, torch)[0])
        plans = [SyncPlan([sp], eng.plan.opt_kind) for sp in eng.plan.spans]
        args = eng.step_args()

        def many(_):
            for p in plans:
                p.run(args)
        key = "one_launch_per_tensor" if per_tensor else "one_launch_per_bucket"
        out[key] = dict(launches=len(plans), spans=len(plans), ms=timed_region(many, max(3, steps // 5), 3, torch)[0])
        del eng, plans
        torch.cuda.empty_cache()
    return out


def reference_profile_metrics(device, steps, torch):
    """The two figures of this path that the reference itself records (IIDPTrainer.profile_step, written to
    examples/resnet50/quickstart/cluster_comp_profile_data/*/*/resnet50_*_comp_profile.json:1): ``update_time`` =
    the optimizer step over the main VSW's parameters, ``copy_time`` = the copy of the main VSW's weights to the
    other K - 1 VSWs, ResNet-50, SGD with momentum, K = 1..4. Here the step is ShardSGD.step() over the 161
    tensors (one planned launch) and the copy is part of that launch (``attach_replicas``): update_time_ms is the
    launch without replicas, copy_time_ms what K - 1 replicas add to it. Beside them, on the same GPU, the
    reference's own structure with stock torch: torch.optim.SGD's single-tensor loop and one ``copy_`` per
    parameter and replica (jabas/train/trainer.py:530-534). ms per call, HIP events, gradients in place."""
    from jabas_amd import workloads as W
    from jabas_amd import optim
    cfg = W.config("resnet50")
    hp = dict(lr=cfg.opt["groups"][0]["lr"], momentum=cfg.opt["momentum"])

    def params(seed):
        gen = torch.Generator(device=device).manual_seed(seed)
        return [torch.nn.Parameter(torch.randn(s.numel, generator=gen, device=device) * 0.05) for s in cfg.specs]

    def groups(ps):
        return [dict(params=[p for p, s in zip(ps, cfg.specs) if s.group == gi], weight_decay=g["weight_decay"])
                for gi, g in enumerate(cfg.opt["groups"])]

    out, base = {}, None
    for K in (1, 2, 3, 4):
        main, stock = params(1), params(1)
        for ps in (main, stock):
            for p in ps:
                p.grad = torch.randn_like(p) * cfg.grad_std
        replicas = [[torch.nn.Parameter(p.detach().clone()) for p in main] for _ in range(K - 1)]
        stock_replicas = [[torch.nn.Parameter(p.detach().clone()) for p in stock] for _ in range(K - 1)]
        mine = optim.ShardSGD(groups(main), **hp)
        if replicas:
            mine.attach_replicas(main, *replicas)
        theirs = torch.optim.SGD(groups(stock), foreach=False, **hp)

        def copy_loop(_):
            with torch.no_grad():
                for rep_ in stock_replicas:
                    for src, dst in zip(stock, rep_):
                        dst.data.copy_(src.data)

        n = max(10, steps)
        fused = timed_region(lambda i: mine.step(), n, 5, torch)[0]
        update_stock = timed_region(lambda i: theirs.step(), max(5, n // 5), 2, torch)[0]
        copy_stock = timed_region(copy_loop, max(5, n // 5), 2, torch)[0] if K > 1 else 0.0
        if K == 1:
            base = fused
        out[str(K)] = dict(update_time_ms=base, copy_time_ms=max(0.0, fused - base), update_and_copy_one_launch_ms=fused,
                           stock_torch_update_time_ms=update_stock, stock_torch_copy_time_ms=copy_stock)
        del main, stock, replicas, stock_replicas, mine, theirs
        torch.cuda.empty_cache()
    return dict(model="resnet50", optimizer="sgd momentum 0.9", tensors=len(cfg.specs),
                elements=sum(s.numel for s in cfg.specs), per_K=out)


def cpu_baseline(cfg, torch, budget_s):
    """Reference-structured unfused step on the host cores: 1 warm-up step (allocates the optimizer state),
    then at least 3 whole steps and as many more as fit about budget_s, all threads; then the same step
    on one thread (bounded)."""
    from jabas_amd.layout import FlatLayout
    from oracle.unfused_baseline import UnfusedStep
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    layout = FlatLayout(cfg.specs)
    numel = sum(s.numel for s in cfg.specs)
    st = UnfusedStep(layout, cfg.batches, gdt, cfg.grad_std, cfg.opt)
    t0 = time.perf_counter()
    st.step(cfg.stats)
    first = time.perf_counter() - t0
    iters = int(max(3, min(8, (budget_s - first) / max(first, 1e-3))))
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        st.step(cfg.stats)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    bytes_per_step = numel * algorithmic_bytes_per_elem(cfg)
    threads = torch.get_num_threads()
    torch.set_num_threads(1)
    one = []
    try:
        t_begin = time.perf_counter()
        while len(one) < 2 and (not one or time.perf_counter() - t_begin + one[-1] < budget_s / 3):
            t0 = time.perf_counter()
            st.step(cfg.stats)
            one.append(time.perf_counter() - t0)
    finally:
        torch.set_num_threads(threads)
    one_best = min(one)
    return dict(value=bytes_per_step / 1e9 / med, unit="GB/s", cores=threads, kind="port",
                ms_per_step=med * 1e3, ms_per_step_min=times[0] * 1e3, ms_per_step_max=times[-1] * 1e3, steps=iters,
                one_thread=dict(value=bytes_per_step / 1e9 / one_best, unit="GB/s", cores=1,
                                ms_per_step=one_best * 1e3, steps=len(one)),
                sample=f"{cfg.name} full gradient set ({numel} elements), unfused torch CPU ops "
                       f"(K in-place aggregate passes, per-bucket clone+scale, cat + cosine_similarity, "
                       f"torch.optim single-tensor loop), median of {iters} whole steps after 1 warm-up")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="vit_l16")
    ap.add_argument("--no-all", action="store_true", help="time only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-extras", action="store_true",
                    help="per workload only the timed steps and the instrumented launches (a kernel trace of such a "
                         "run holds one kind of launch per kernel name and grid)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0,
                    help="CPU time the headline's baseline may take; the other workloads get a third each")
    ap.add_argument("--bucket-launches", type=int, default=0, metavar="S",
                    help="run only this: the headline workload's gradient set as one launch per bucket, bucket i on "
                         "launch stream i mod S, --steps steps after --warmup (for a kernel trace of the launches)")
    ap.add_argument("--flat-moments", action="store_true",
                    help="keep Adam's moments in flat arenas of their own (the layout before the interleaved moment "
                         "arena, sync.MomentArena) in every engine this run builds: for A/B runs of the two layouts")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB copy 5 times before anything else (the K=1, weight-1 aggregate: "
                         "same 16-byte nontemporal loads and stores as the fused kernel, known traffic) for "
                         "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    global FLAT_MOMENTS
    FLAT_MOMENTS = bool(args.flat_moments)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures the one-GPU share of the gradient-sync path; "
                 "run it with --gpus 1 (no collectives are part of the path)")
    import torch
    from jabas_amd import workloads as W
    from jabas_amd import _lib
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a GPU (the HIP path has no CPU fallback)")
    _lib.lib()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    head_cfg = W.config(args.workload)
    if args.calibrate_copy:
        from jabas_amd import sync
        src = torch.ones(1 << 28, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        for _ in range(5):
            sync.aggregate([src], (1,), out=dst)       # fused_kernel<1, f32, none, no stats>: out = src * 1.0f
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    if args.bucket_launches:
        engines, numel, _ = build_engines(head_cfg, device, torch)
        ms = bucket_launches(head_cfg, engines[0], device, args.steps, args.warmup, torch, args.bucket_launches)
        print(json.dumps(dict(workload=head_cfg.name, launch_streams=args.bucket_launches, steps=args.steps,
                              buckets=engines[0].plan.n_span, **rate(numel * algorithmic_bytes_per_elem(head_cfg), ms))))
        return
    results, failures = {}, {}

    def guarded(label, fn):
        """A leg beside the headline that raises is named in the line ("failures") instead of taking the line with it."""
        try:
            return fn()
        except Exception as exc:
            failures[label] = f"{type(exc).__name__}: {exc}"
            print(f"# {label} failed: {failures[label]}", file=sys.stderr, flush=True)
            try:
                torch.cuda.synchronize()
                torch.cuda.empty_cache()
            except Exception:
                pass
            return None

    order = [head_cfg] + ([] if args.no_all else [c for c in W.configs() if c.name != head_cfg.name])
    for cfg in list(order):
        r = None
        if not args.no_extras:
            r = guarded(f"{cfg.name} with its extra legs",
                        lambda: time_config(cfg, device, args.steps, args.warmup, torch, extras=True))
        if r is None:                               # the step alone; the headline's own failure is the bench's
            if cfg is head_cfg:
                r = time_config(cfg, device, args.steps, args.warmup, torch, extras=False)
            else:
                r = guarded(cfg.name, lambda: time_config(cfg, device, args.steps, args.warmup, torch, extras=False))
        if r is None:
            order.remove(cfg)
            continue
        results[cfg.name] = r
        r["hbm_traffic_bytes_per_launch"] = measured_traffic(cfg.name)
        if args.no_extras or "hook_path_per_bucket_ms" not in r:
            print(f"# {cfg.name}: {r['ms_per_step']:.4f} ms/step, {r['GBps']:.0f} GB/s, {r['pct_hbm_peak']:.1f} % of HBM peak",
                  file=sys.stderr, flush=True)
            continue
        extra = ""
        if r.get("step_without_statistics"):
            extra = (f"; without statistics {r['step_without_statistics']['ms_per_step']:.4f} ms "
                     f"{r['step_without_statistics']['pct_hbm_peak']:.1f} %; per-VSW norms too "
                     f"{r['step_with_per_vsw_norms']['pct_hbm_peak']:.1f} %")
        print(f"# {cfg.name}: {r['ms_per_step']:.4f} ms/step, {r['GBps']:.0f} GB/s, "
              f"{r['pct_hbm_peak']:.1f} % of HBM peak{extra}; hooks per bucket "
              f"{r['hook_path_per_bucket_ms']['ms_per_step']:.4f} ms, batched "
              f"{r['hook_path_batched_64MiB_ms']['ms_per_step']:.4f} ms, deferred "
              f"{r['hook_path_deferred_ms']['ms_per_step']:.4f} ms; one launch per bucket back to back on 1 / 2 launch "
              f"streams {r['bucket_launches_back_to_back_ms']['1']:.4f} / {r['bucket_launches_back_to_back_ms']['2']:.4f} ms; "
              f"K hook threads: exposed sync {r['hook_path_threads_2_launch_streams'].get('exposed_sync_ms', float('nan')):.4f} ms",
              file=sys.stderr, flush=True)
    if "faster_rcnn_r50_fpn" in results and not args.no_extras:
        results["faster_rcnn_r50_fpn"]["launch_modes"] = guarded(
            "launch_modes", lambda: launch_modes(W.config("faster_rcnn_r50_fpn"), device, args.steps, torch))
    side = not (args.no_all or args.no_extras)
    ref_metrics = guarded("reference_profile_metrics", lambda: reference_profile_metrics(device, args.steps, torch)) if side else None
    copy_gbps = guarded("copy_rate", lambda: copy_rate(device, args.steps, torch))
    stat_launches = guarded("statistics_launches", lambda: statistics_launches(device, args.steps, torch)) if side else None
    gram = guarded("gram_launches", lambda: gram_launches(device, args.steps, torch)) if side else None
    head = results[head_cfg.name]
    if not args.no_cpu:
        for cfg in order:
            budget = args.cpu_seconds if cfg.name == head_cfg.name else args.cpu_seconds / 3.0
            c = results[cfg.name]["cpu_baseline"] = guarded(f"cpu_baseline {cfg.name}", lambda: cpu_baseline(cfg, torch, budget))
            if c is not None:
                print(f"# cpu {cfg.name}: {c['ms_per_step']:.1f} ms/step on {c['cores']} threads ({c['steps']} steps), "
                      f"{c['one_thread']['ms_per_step']:.1f} ms on one", file=sys.stderr, flush=True)
    bytes_per_launch = head["GB_per_step"] * 1e9
    # one fused-kernel launch per step (plus the statistics' finalize launch, about 1 % of it): the mean
    # launch duration is the HIP-event time of the timed region over its steps
    roofline = dict(bound="hbm", achieved=head["GBps"], peak=HBM_PEAK_GBPS, unit="GB/s",
                    frac=head["GBps"] / HBM_PEAK_GBPS, traffic=head["hbm_traffic_bytes_per_launch"],
                    traffic_source=TRAFFIC_FILE if head["hbm_traffic_bytes_per_launch"] is not None else None,
                    kernel="jabas::fused_kernel", algorithmic_bytes_per_launch=bytes_per_launch,
                    launch_ms=head["ms_per_step"], launch_ms_isolated=head["launch_ms_mean"],
                    copy_GBps=copy_gbps)
    out = {
        "metric": "sync_step_GBps", "value": head["GBps"], "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": head_cfg.name, "elements": head["elements"], "K": head["K"],
                   "batches": head["batches"], "grad_dtype": head["grad_dtype"], "optimizer": head["optimizer"],
                   "stats": head["stats"], "bytes_per_elem": head["bytes_per_elem"],
                   "adam_moments": "flat arenas" if FLAT_MOMENTS else "one arena, interleaved in blocks of 8192 elements"},
        "pct_hbm_peak": head["pct_hbm_peak"],
        "roofline": roofline,
        "cpu_baseline": head.get("cpu_baseline"),
        "copy_GBps": copy_gbps,
        "workloads": list(results.values()),
        "reference_profile_metrics_resnet50": ref_metrics,
        # the configuration an earlier headline was quoted on (ViT-B/16, K = 4, fp32 gradients, full statistics
        # rows), so that figures stay comparable over time whatever the headline workload is
        "like_for_like": {"vit_b16_K4_f32_full_statistics_rows":
                          results.get("vit_b16", {}).get("step_with_per_vsw_norms")},
        "statistics_launches": stat_launches,
        "gram_launches": gram,
        "device": guarded("device_info", lambda: device_info(device, torch)),
        "failures": failures,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
