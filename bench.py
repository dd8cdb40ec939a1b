#!/usr/bin/env python3
"""Benchmark of the fused per-GPU gradient-sync step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-all] [--no-cpu]

A step is one fused sync step (batch-weighted aggregate of the K VSW gradient buckets
+ gradient statistics where the configuration asks for them + optimizer update) over
one full synthetic gradient set. The headline workload is the ViT-B/16 configuration;
the other four configurations are timed too and reported under "workloads" in the
same JSON line. Inputs are resident in HBM before the timed region starts. Small
configurations rotate over several copies of their buffers so that the working set
stays far above the 256 MB last-level cache.

Prints ONE JSON line: metric sync_step_GBps = algorithmic bytes per step / time per step,
with a "roofline" object (HBM-bound; achieved = algorithmic bytes per launch / mean
launch duration from HIP events on the launching stream) and a "cpu_baseline" object
(the reference's unfused PyTorch structure timed on this box's host cores, rank 0 only).
"""
import argparse
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

# HBM bytes per launch of the fused kernel measured with rocprofv3 --pmc (FETCH_SIZE and
# WRITE_SIZE runs, scaled by a copy kernel of known size; profiles/fused_kernel_hbm_traffic_pmc.md).
MEASURED_TRAFFIC_BYTES = {"vit_b16": 3816.9e6, "resnet50": 718.9e6, "faster_rcnn_r50_fpn": 1345.5e6,
                          "gnmt": 7083.6e6, "vit_l16": 13405.5e6}


def algorithmic_bytes_per_elem(cfg):
    s_g = 2 if cfg.grad_dtype == "bf16" else 4
    state = 16 if cfg.opt["kind"] == "sgd" else 24
    return cfg.K * s_g + 4 + state


def build_engines(cfg, device, torch):
    from jabas_amd.engine import VSWFlatSync
    from jabas_amd import workloads as W
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    numel = sum(s.numel for s in cfg.specs)
    ws = numel * algorithmic_bytes_per_elem(cfg)
    copies = max(1, math.ceil(ROTATE_TARGET_BYTES / ws))
    engines = []
    for c in range(copies):
        eng = VSWFlatSync(cfg.specs, cfg.batches, grad_dtype=gdt, opt=cfg.opt, device=device)
        gen = torch.Generator(device=device).manual_seed(1234 + 17 * c)
        for k in range(cfg.K):
            tmp = torch.randn(eng.layout.total, generator=gen, device=device, dtype=torch.float32) * cfg.grad_std
            eng.grads[k].copy_(tmp.to(gdt))
            del tmp
        eng.param.copy_(torch.randn(eng.layout.total, generator=gen, device=device) * 0.05)
        if cfg.name == "gnmt":
            # embedding gradient: a fixed random 10 % of the rows non-zero, same rows for every VSW
            i = [s.name for s in cfg.specs].index(W.GNMT_EMBEDDING)
            rows, cols = W.GNMT_EMBEDDING_ROWS, W.GNMT_EMBEDDING_COLS
            keep = (torch.rand(rows, generator=torch.Generator().manual_seed(0)) < 0.1).to(device)
            for k in range(cfg.K):
                v = eng.grad_view(k, i).view(rows, cols)
                v.copy_(torch.where(keep[:, None], v, torch.zeros((), device=device, dtype=v.dtype)))
        engines.append(eng)
    return engines, numel, copies


def time_config(cfg, device, steps, warmup, torch):
    engines, numel, copies = build_engines(cfg, device, torch)
    bytes_per_step = numel * algorithmic_bytes_per_elem(cfg)
    n = len(engines)
    for i in range(warmup):
        engines[i % n].step(stats=cfg.stats)
    torch.cuda.synchronize()
    # timed region: exactly `steps` steps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        engines[i % n].step(stats=cfg.stats)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    region_ms = e0.elapsed_time(e1)
    ms_per_step = max(region_ms, 1e-6) / steps
    # per-launch durations (instrumentation pass, outside the timed region)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i, (a, b) in enumerate(evs):
        a.record()
        engines[i % n].step(stats=cfg.stats)
        b.record()
    torch.cuda.synchronize()
    launch_ms = sorted(a.elapsed_time(b) for a, b in evs)
    mean_launch_ms = sum(launch_ms) / len(launch_ms)
    # the step between statistic steps (statistics run every `interval` steps in training): same
    # bytes, no fp64 sums, the launch shape of the plain kernels
    plain = None
    if cfg.stats:
        for i in range(warmup):
            engines[i % n].step(stats=False)
        p0, p1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        p0.record()
        for i in range(steps):
            engines[i % n].step(stats=False)
        p1.record()
        torch.cuda.synchronize()
        plain_ms = max(p0.elapsed_time(p1), 1e-6) / steps
        plain = dict(ms_per_step=plain_ms, GBps=bytes_per_step / 1e9 / (plain_ms / 1e3),
                     pct_hbm_peak=100.0 * bytes_per_step / 1e9 / (plain_ms / 1e3) / HBM_PEAK_GBPS)
    stats_rows = engines[0].step(stats=True) if cfg.stats else None
    cos = engines[0].cosine(stats_rows) if stats_rows is not None else None
    finite = bool(torch.isfinite(engines[0].param).all())
    res = dict(
        workload=cfg.name, elements=numel, K=cfg.K, batches=list(cfg.batches), grad_dtype=cfg.grad_dtype,
        optimizer=cfg.opt["kind"], stats=cfg.stats, spans=engines[0].plan.n_span,
        bytes_per_elem=algorithmic_bytes_per_elem(cfg), GB_per_step=bytes_per_step / 1e9,
        ms_per_step=ms_per_step, wall_ms_per_step=wall_ms / steps, GBps=bytes_per_step / 1e9 / (ms_per_step / 1e3),
        launch_ms_mean=mean_launch_ms, launch_ms_median=launch_ms[len(launch_ms) // 2], launch_ms_min=launch_ms[0],
        GBps_launch=bytes_per_step / 1e9 / (mean_launch_ms / 1e3),
        pct_hbm_peak=100.0 * bytes_per_step / 1e9 / (mean_launch_ms / 1e3) / HBM_PEAK_GBPS,
        buffer_copies=copies, cosine=cos, finite=finite, step_without_statistics=plain)
    del engines
    torch.cuda.empty_cache()
    return res


def launch_modes(cfg, device, steps, torch):
    """Small-span launch overhead (the Faster R-CNN configuration's point): the same step as
    one launch over bucket spans, one launch over one span per tensor, one launch per
    bucket, and one launch per tensor. ms per step from HIP events."""
    from jabas_amd.engine import VSWFlatSync
    from jabas_amd.sync import SyncPlan
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    out = {}

    def timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    for label, per_tensor in (("one_launch_bucket_spans", False), ("one_launch_tensor_spans", True)):
        eng = VSWFlatSync(cfg.specs, cfg.batches, grad_dtype=gdt, opt=cfg.opt, device=device, per_tensor_spans=per_tensor)
        for g in eng.grads:
            g.normal_(0, cfg.grad_std)
        eng.param.normal_(0, 0.05)
        eng.step()
        out[label] = dict(launches=1, spans=eng.plan.n_span, ms=timed(lambda: eng.step(), steps))
        plans = [SyncPlan([sp], eng.plan.opt_kind) for sp in eng.plan.spans]
        args = eng.step_args()

        def many():
            for p in plans:
                p.run(args)
        key = "one_launch_per_tensor" if per_tensor else "one_launch_per_bucket"
        out[key] = dict(launches=len(plans), spans=len(plans), ms=timed(many, max(3, steps // 5)))
        del eng, plans
        torch.cuda.empty_cache()
    return out


def cpu_baseline(cfg, torch, budget_s=25.0):
    """Reference-structured unfused step on the host cores, bounded to about budget_s."""
    from jabas_amd.layout import FlatLayout
    from oracle.unfused_baseline import UnfusedStep
    gdt = torch.bfloat16 if cfg.grad_dtype == "bf16" else torch.float32
    layout = FlatLayout(cfg.specs)
    numel = sum(s.numel for s in cfg.specs)
    st = UnfusedStep(layout, cfg.batches, gdt, cfg.grad_std, cfg.opt)
    t0 = time.perf_counter()
    st.step(cfg.stats)                                 # warm-up (allocates optimizer state)
    first = time.perf_counter() - t0
    iters = int(max(2, min(8, (budget_s - first) / max(first, 1e-3))))
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        st.step(cfg.stats)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    bytes_per_step = numel * algorithmic_bytes_per_elem(cfg)
    # the same step on one host thread (bounded: at most 3 steps or ~10 s)
    threads = torch.get_num_threads()
    torch.set_num_threads(1)
    one = []
    try:
        t_begin = time.perf_counter()
        while len(one) < 3 and (not one or time.perf_counter() - t_begin + one[-1] < 10.0):
            t0 = time.perf_counter()
            st.step(cfg.stats)
            one.append(time.perf_counter() - t0)
    finally:
        torch.set_num_threads(threads)
    one_best = min(one)
    return dict(value=bytes_per_step / 1e9 / med, unit="GB/s", cores=threads, kind="port",
                ms_per_step=med * 1e3,
                one_thread=dict(value=bytes_per_step / 1e9 / one_best, unit="GB/s", cores=1,
                                ms_per_step=one_best * 1e3, steps=len(one)),
                sample=f"{cfg.name} full gradient set ({numel} elements), unfused torch CPU ops "
                       f"(K in-place aggregate passes, per-bucket clone+scale, cat + cosine_similarity, "
                       f"torch.optim single-tensor loop), median of {iters} steps after 1 warm-up")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="vit_b16")
    ap.add_argument("--no-all", action="store_true", help="time only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB copy 5 times (the K=1, weight-1 aggregate: same 16-byte "
                         "nontemporal loads and stores as the fused kernel, known traffic) for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
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
    results = {}
    order = [head_cfg] + ([] if args.no_all else [c for c in W.configs() if c.name != head_cfg.name])
    for cfg in order:
        results[cfg.name] = time_config(cfg, device, args.steps, args.warmup, torch)
        r = results[cfg.name]
        extra = ""
        if r["step_without_statistics"]:
            extra = (f"; without statistics {r['step_without_statistics']['ms_per_step']:.4f} ms/step, "
                     f"{r['step_without_statistics']['pct_hbm_peak']:.1f} %")
        print(f"# {cfg.name}: {r['ms_per_step']:.4f} ms/step, {r['GBps']:.0f} GB/s, "
              f"{r['pct_hbm_peak']:.1f} % of HBM peak{extra}", file=sys.stderr, flush=True)
    if "faster_rcnn_r50_fpn" in results:
        results["faster_rcnn_r50_fpn"]["launch_modes"] = launch_modes(W.config("faster_rcnn_r50_fpn"), device,
                                                                      args.steps, torch)
    head = results[head_cfg.name]
    bytes_per_launch = head["GB_per_step"] * 1e9
    roofline = dict(bound="hbm", achieved=head["GBps_launch"], peak=HBM_PEAK_GBPS, unit="GB/s",
                    frac=head["GBps_launch"] / HBM_PEAK_GBPS,
                    traffic=MEASURED_TRAFFIC_BYTES.get(head_cfg.name),
                    kernel="jabas::fused_kernel", algorithmic_bytes_per_launch=bytes_per_launch,
                    launch_ms=head["launch_ms_mean"])
    cpu = None if args.no_cpu else cpu_baseline(head_cfg, torch)
    out = {
        "metric": "sync_step_GBps", "value": head["GBps"], "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": head_cfg.name, "elements": head["elements"], "K": head["K"],
                   "batches": head["batches"], "grad_dtype": head["grad_dtype"], "optimizer": head["optimizer"],
                   "stats": head["stats"], "bytes_per_elem": head["bytes_per_elem"]},
        "pct_hbm_peak": head["pct_hbm_peak"],
        "roofline": roofline,
        "cpu_baseline": cpu,
        "workloads": list(results.values()),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
