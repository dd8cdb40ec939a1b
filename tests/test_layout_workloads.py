"""Bucket layout and workload shape checks (CPU)."""
import json
import os

import pytest
import torch
import torch.distributed as dist

from jabas_amd import layout as L
from jabas_amd import workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))


def test_workload_element_counts_match_the_benchmark_specification():
    want = {"resnet50": (161, 25_557_032), "vit_b16": (152, 86_567_656), "gnmt": (44, 160_665_150),
            "vit_l16": (296, 304_326_632)}
    for name, (tensors, elems) in want.items():
        specs = W.config(name).specs
        assert len(specs) == tensors and sum(s.numel for s in specs) == elems, name
    frcnn = W.config("faster_rcnn_r50_fpn").specs
    assert len(frcnn) == 280 and 40e6 < sum(s.numel for s in frcnn) < 43e6
    assert [c.K for c in W.configs()] == [2, 4, 3, 4, 8]
    assert W.config("vit_l16").batches == (64, 56, 48, 40, 32, 24, 16, 8)


def test_resnet50_buckets_match_the_reference_profile_fixture():
    """Known answer held by the reference: the DDP bucket sizes its bucket profiler recorded
    for ResNet-50 (MiB). The recorded run bucketed in true gradient-ready order, the helper
    in reverse registration order: same cut points, sizes within 0.1 MiB."""
    fixture = json.load(open(os.path.join(HERE, "golden", "resnet50_bucket_size_profile.json")))
    got = L.FlatLayout(W.resnet50()).bucket_sizes_mb()
    want = fixture["bucket_size_distribution"]
    assert len(got) == len(want) == 5
    for g, w in zip(got, want):
        assert abs(g - w) <= 0.1, (got, want)
    assert abs(sum(got) - sum(want)) <= 0.2


@pytest.mark.parametrize("name", ["resnet50", "vit_b16", "gnmt", "faster_rcnn_r50_fpn"])
def test_bucket_assignment_equals_torch_ddp_rule(name):
    specs = W.config(name).specs
    numels = [s.numel for s in specs]
    mine = L.bucket_assignment(numels)
    metas = [torch.empty(n, device="meta") for n in reversed(numels)]
    theirs, _ = dist._compute_bucket_assignment_by_size(metas, [1 << 20, 25 << 20])
    n = len(numels)
    assert [[n - 1 - i for i in b] for b in theirs] == mine


def test_flat_layout_is_a_packed_partition_with_consistent_bounds():
    specs = W.vit_b16()
    lay = L.FlatLayout(specs)
    seen = set()
    for b in lay.buckets:
        assert b.offset % L.BUCKET_ALIGN_ELEMS == 0
        pos = b.offset
        for i in b.param_ids:
            assert lay.param_offset[i] == pos and lay.param_bucket[i] == b.index
            pos += specs[i].numel
            seen.add(i)
        assert pos == b.offset + b.numel
        assert b.bounds[0][0] == 0
        starts = [s for s, _ in b.bounds]
        assert starts == sorted(set(starts))
        for (s0, g0), (s1, g1) in zip(b.bounds, b.bounds[1:]):
            assert g0 != g1                                   # adjacent stretches of one group are merged
        # every tensor's group is the group of the stretch it lies in
        for i in b.param_ids:
            rel = lay.param_offset[i] - b.offset
            grp = [g for s, g in b.bounds if s <= rel][-1]
            assert grp == specs[i].group
    assert seen == set(range(len(specs)))
    assert lay.numel == sum(s.numel for s in specs) and lay.total >= lay.numel


def test_per_tensor_spans_cover_every_tensor_once():
    specs = W.faster_rcnn_r50_fpn()
    lay = L.FlatLayout(specs, per_tensor_spans=True)
    assert len(lay.spans) == len(specs)
    assert sum(n for _, n, _, _ in lay.spans) == lay.numel


def test_tracked_hbm_traffic_covers_every_workload_at_its_algorithmic_bytes():
    """bench.py's roofline.traffic is read from a tracked summary of two rocprofv3 counter runs: it must name every
    workload the package defines, at the algorithmic bytes bench.py prices that workload with (a workload whose
    shape or byte count moved needs the counters taken again), and the traffic may not be below the algorithmic
    bytes nor more than a few per cent above."""
    import json
    import os
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    import bench
    from jabas_amd import workloads as W
    with open(os.path.join(root, bench.TRAFFIC_FILE)) as f:
        table = json.load(f)["workloads"]
    for cfg in W.configs():
        assert cfg.name in table, f"{bench.TRAFFIC_FILE} lacks {cfg.name}"
        want = sum(s.numel for s in cfg.specs) * bench.algorithmic_bytes_per_elem(cfg)
        entry = table[cfg.name]
        assert abs(entry["algorithmic_bytes"] - want) <= 1e-5 * want, (cfg.name, entry["algorithmic_bytes"], want)
        assert 1.0 <= entry["hbm_bytes_per_launch"] / want <= 1.02, cfg.name
        assert bench.measured_traffic(cfg.name) == entry["hbm_bytes_per_launch"]
