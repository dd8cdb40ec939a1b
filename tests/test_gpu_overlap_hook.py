"""GPU parity of the overlap weight-sync mode (jabas/train/trainer.py:327-333): the optimizer hook on
VSW 0. K hook threads on K streams publish their buckets; the fused launch of a bucket (queued by the
last VSW to arrive, on a launch stream of its own) aggregates, updates the weights of that bucket's
parameters and refreshes the other replicas. Everything is compared bit for bit with the CPU oracle's
``sync_step`` over several steps: aggregate, weights, optimizer state, replica weights.
VSW 0 publishes FIRST in every case, so an update that ran at VSW 0's hook time would see its own
un-aggregated bucket and fail here.
"""
import math
import threading

import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({8: torch.int64, 4: torch.int32, 2: torch.int16}[t.element_size()])


def _same(a, b):
    return torch.equal(_bits(a.reshape(-1)), _bits(b.reshape(-1)))


class ParamBucket:
    """What a comm hook is handed: index(), buffer(), parameters(), gradients() (views of the buffer)."""

    def __init__(self, i, buf, params, offs):
        self._i, self._buf, self._params, self._offs = i, buf, params, offs

    def index(self):
        return self._i

    def buffer(self):
        return self._buf

    def parameters(self):
        return list(self._params)

    def gradients(self):
        return [self._buf[o:o + p.numel()].view(p.shape) for p, o in zip(self._params, self._offs)]


# three buckets; 1-D tensors (group 0: no weight decay) and matrices (group 1) alternate, odd sizes so
# that group changes fall inside 16-byte vectors and tiles
SHAPES = [[(33,), (129, 61), (61,), (70, 70)], [(5,)], [(300, 257), (257,), (3, 3), (9,), (1000, 41)]]


def _opt_dict(kind):
    if kind == "sgd":
        return dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                    groups=[dict(lr=0.1, weight_decay=0.0), dict(lr=0.1, weight_decay=1e-4)])
    return dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8, amsgrad=kind.endswith("amsgrad"),
                groups=[dict(lr=5e-4, weight_decay=0.0), dict(lr=5e-4, weight_decay=0.05)])


def _torch_optimizer(kind, params):
    groups = [{"params": [p for p in params if p.dim() <= 1], "weight_decay": 0.0},
              {"params": [p for p in params if p.dim() > 1], "weight_decay": 1e-4 if kind == "sgd" else 0.05}]
    if kind == "sgd":
        return torch.optim.SGD(groups, lr=0.1, momentum=0.9)
    return torch.optim.AdamW(groups, lr=5e-4, amsgrad=kind.endswith("amsgrad"))


def _layout(shapes):
    offs, bounds, o = [], [], 0
    for s in shapes:
        n = math.prod(s)
        g = 0 if len(s) <= 1 else 1
        if not bounds or bounds[-1][1] != g:
            bounds.append((o if bounds else 0, g))
        offs.append(o)
        o += n
    return offs, tuple(bounds), o


@pytest.mark.parametrize("kind", ["sgd", "adamw"])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["per_bucket", "deferred", "batched"])
def test_optimizer_in_the_hook_is_bit_exact_with_the_oracle(gpu, kind, gdt, mode):
    _hooks_with_optimizer(gpu, kind, gdt, mode, (4, 2, 2))


@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["per_bucket", "deferred"])
def test_optimizer_in_the_hook_with_amsgrad(gpu, gdt, mode):
    """AdamW(amsgrad=True) bound to the hooks: the running maximum lives in a third state arena laid out like
    the bucket, ``optimizer.state[p]['max_exp_avg_sq']`` shows it."""
    _hooks_with_optimizer(gpu, "adamw_amsgrad", gdt, mode, (4, 2, 2))


@pytest.mark.parametrize("kind", ["adamw", "adamw_amsgrad"])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["per_bucket", "deferred", "batched"])
def test_optimizer_in_the_hook_with_interleaved_moments(gpu, kind, gdt, mode):
    """``LocalBucketSync(interleave_moments=True)``: the moments of a bucket's parameters in one arena of alternating
    blocks; weights bit-exact as with flat arenas, the moments bit-exact in what ``optimizer.state_dict()`` shows,
    ``optimizer.state[p]`` without them in between."""
    _hooks_with_optimizer(gpu, kind, gdt, mode, (4, 2, 2), launch_streams=2, interleave=True)


@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
def test_overlap_mode_that_writes_no_aggregate(gpu, gdt):
    """``write_aggregate=False``: weights, state and replicas as before, VSW 0's bucket left as backward filled
    it, no fp32 arena beside reduced-precision buckets."""
    _hooks_with_optimizer(gpu, "adamw", gdt, "per_bucket_no_aggregate", (4, 2, 2))


@pytest.mark.parametrize("kind", ["sgd", "adamw"])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode,launch_streams", [("per_bucket", 2), ("per_bucket", 3), ("batched", 2)])
def test_launches_alternating_between_launch_streams(gpu, kind, gdt, mode, launch_streams):
    """Consecutive buckets' launches on alternating launch streams (they overlap on the GPU): the same bits."""
    _hooks_with_optimizer(gpu, kind, gdt, mode, (4, 2, 2), launch_streams=launch_streams)


@pytest.mark.parametrize("kind", ["sgd", "adamw"])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["per_bucket", "batched", "deferred"])
def test_launches_on_the_stream_of_the_vsw_that_came_last(gpu, kind, gdt, mode):
    """``launch_on_last_vsw``: no stream beside the VSWs' own; VSW 0 always hands over first here, so every
    launch sits on a peer's stream behind an event from VSW 0's. The same bits, and the second and third step
    through the native meeting point."""
    _hooks_with_optimizer(gpu, kind, gdt, mode, (4, 2, 2), launch_streams=0)


# buckets of 8, 12 and 17 MB: a bucket's launch is still running when the next bucket is handed over
BIG_SHAPES = [[(1024, 2048), (2048,)], [(1536, 2048), (7,)], [(2048, 1024), (1024,), (1100, 2000)]]


@pytest.mark.parametrize("gdt,launch_streams", [(torch.float32, 1), (torch.bfloat16, 2), (torch.float32, 0)])
def test_multi_megabyte_buckets_through_the_native_meeting_point(gpu, gdt, launch_streams):
    """K = 4 hook threads, buckets large enough that launches are in flight at the following hand-overs; the
    second and third step go through the native meeting point."""
    _hooks_with_optimizer(gpu, "adamw", gdt, "per_bucket", (48, 32, 32, 16), launch_streams=launch_streams,
                          SHAPES=BIG_SHAPES)


@pytest.mark.parametrize("mode,launch_streams", [("per_bucket", 1), ("batched", 1), ("per_bucket", 0)])
def test_eight_vsw_threads_with_bf16_buckets(gpu, mode, launch_streams):
    """The largest configuration's shape: eight VSWs with batches 64..8, bf16 buckets, AdamW."""
    _hooks_with_optimizer(gpu, "adamw", torch.bfloat16, mode, (64, 56, 48, 40, 32, 24, 16, 8),
                          launch_streams=launch_streams)


def _checkpointed(optimizer):
    """id(parameter) -> its entry of ``optimizer.state_dict()["state"]``: the state as a checkpoint sees it."""
    sd = optimizer.state_dict()
    params = [p for g in optimizer.param_groups for p in g["params"]]
    index = [i for g in sd["param_groups"] for i in g["params"]]
    return {id(p): sd["state"][i] for p, i in zip(params, index) if i in sd["state"]}


def _hooks_with_optimizer(gpu, kind, gdt, mode, batches, launch_streams=1, SHAPES=SHAPES, interleave=False):
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    from jabas_amd.train import create_optimizer_hook, create_stream_for_optimizer

    K = len(batches)
    opt = _opt_dict(kind)
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    # K replicas of the "model": one Parameter per tensor, the same initial values
    gen = torch.Generator().manual_seed(5)
    init = [[torch.randn(s, generator=gen) * 0.05 for s in shapes] for shapes in SHAPES]
    replicas = [[[torch.nn.Parameter(t.clone().to(gpu)) for t in bucket] for bucket in init] for _ in range(K)]
    layouts = [_layout(shapes) for shapes in SHAPES]
    bufs = [[torch.zeros(n, dtype=gdt, device=gpu) for _ in range(K)] for (_, _, n) in layouts]
    optimizer = _torch_optimizer(kind, [p for bucket in replicas[0] for p in bucket])
    # batched: complete buckets wait until 400 kB of them are ready, then go out as one planned launch
    keep = not mode.endswith("no_aggregate")
    mode = mode.replace("_no_aggregate", "")
    # launch_streams=0: no launch stream at all, a bucket's launch on the stream of the VSW that completed it
    local = LocalBucketSync(batches, deferred=(mode == "deferred"), batch_bytes=400_000 if mode == "batched" else 0,
                            stream=create_stream_for_optimizer(gpu) if launch_streams else None, write_aggregate=keep,
                            launch_streams=launch_streams, interleave_moments=interleave,
                            launch_on_last_vsw=not launch_streams)
    assert len(local._sync_streams) == launch_streams
    st = H.GradientSimilarityState(None, K + K % 2, None, [], 2).attach_local(local)
    main_hook = create_optimizer_hook(H.similimarity_allreduce_hook(H.subgroup_allreduce_hook), optimizer)
    # the oracle's flat state per bucket
    p_h = [torch.cat([t.reshape(-1) for t in bucket]) for bucket in init]
    s1_h = [torch.zeros_like(p) for p in p_h]
    s2_h = [torch.zeros_like(p) for p in p_h]
    s3_h = [torch.zeros_like(p) if kind.endswith("amsgrad") else None for p in p_h]
    gate = [threading.Event() for _ in range(len(SHAPES))]
    for step in range(1, 4):
        local.lr_scale = (1.0, math.sqrt(20 / 8), 0.75)[step - 1]              # the adaptive-batching modifier moves
        std = 1e-3 if step == 1 or not kind.endswith("amsgrad") else 5e-5     # amsgrad: the moment falls below its maximum
        host = [[(torch.randn(n, generator=torch.Generator().manual_seed(1000 * step + 10 * b + k)) * std).to(gdt)
                 for k in range(K)] for b, (_, _, n) in enumerate(layouts)]
        for g in gate:
            g.clear()
        errors = []

        def vsw(k):
            try:
                with torch.cuda.stream(streams[k]):
                    order = range(len(SHAPES)) if k % 2 == 0 else reversed(range(len(SHAPES)))
                    for b in order:
                        if k != 0:
                            gate[b].wait(30)                                    # VSW 0 always hands its bucket over first
                        bufs[b][k].copy_(host[b][k].to(gpu))                    # "backward" fills the bucket on this stream
                        bucket = ParamBucket(b, bufs[b][k], replicas[k][b], layouts[b][0])
                        if k == 0:
                            main_hook(st, bucket).wait()
                            gate[b].set()
                        else:
                            H.dummy_hook(H.VSWPeerState(local, k), bucket).wait()
            except Exception as exc:                                            # pragma: no cover - reported below
                errors.append(exc)
                for g in gate:
                    g.set()

        threads = [threading.Thread(target=vsw, args=(k,), daemon=True) for k in range(K)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(60)
        assert not errors, errors
        local.finish_step()
        torch.cuda.synchronize()
        want_stats = st.step % st.interval == 0
        # interleaved moments: the optimizer object holds them only while its state_dict() is made
        seen = _checkpointed(optimizer) if interleave else None
        for b, (offs, bounds, n) in enumerate(layouts):
            agg_h, rows_h = O.sync_step(host[b], batches, [(0, n, bounds)], opt, p_h[b], s1_h[b], s2_h[b], step=step,
                                        first_step=(step == 1), want_stats=want_stats, lr_scale=local.lr_scale,
                                        state3=s3_h[b])
            agg_d = bufs[b][0] if gdt == torch.float32 else local.aggregate_of(b)
            if keep:
                assert _same(agg_d, agg_h), (step, b, "aggregate")
            else:
                assert _same(bufs[b][0], host[b][0]) and local.aggregate_of(b) is None
            for i, (p, o) in enumerate(zip(replicas[0][b], offs)):
                sl = slice(o, o + p.numel())
                assert _same(p.data, p_h[b][sl]), (step, b, i, "weights")
                state = optimizer.state[p]
                if interleave and kind != "sgd":
                    assert "exp_avg" not in state and int(state["step"]) == step
                    state = seen[id(p)]
                if kind == "sgd":
                    assert _same(state["momentum_buffer"], s1_h[b][sl]), (step, b, i, "momentum")
                else:
                    assert _same(state["exp_avg"], s1_h[b][sl]) and _same(state["exp_avg_sq"], s2_h[b][sl]), (step, b, i)
                    assert int(state["step"]) == step
                    if kind.endswith("amsgrad"):
                        assert _same(state["max_exp_avg_sq"], s3_h[b][sl]), (step, b, i, "maximum")
                for k in range(1, K):
                    assert _same(replicas[k][b][i].data, p.data), (step, b, i, k, "replica")
            for k in range(1, K):                                               # the peers' buckets are only read
                assert _same(bufs[b][k], host[b][k])
        if want_stats:
            rows = {s.index: s.cpu() for s in st.grad_placeholder}
            assert sorted(rows) == list(range(len(SHAPES)))
            for b, (_, _, n) in enumerate(layouts):
                want = O.stats(host[b], batches)
                tol = 1e-6 if gdt == torch.float32 else 1e-2
                assert torch.allclose(rows[b][1:4], want[1:4], rtol=tol, atol=0.0)
                assert abs(float(rows[b][0] - want[0])) <= tol * float(torch.sqrt(want[1] * want[2]))
                assert torch.count_nonzero(rows[b][4:]) == 0                # the hooks ask for the similarity sums only
        else:
            assert st.grad_placeholder == []
        st.grad_placeholder.clear()
        st.step += 1
    if mode == "batched":
        assert 3 * 1 <= local.launched <= 3 * len(SHAPES)
    else:
        assert local.launched == 3 * (1 if mode == "deferred" else len(SHAPES))
    # one launch per bucket: the first step describes the buckets to the native meeting point, the hand-overs of
    # the second (a statistics step) and third go through it
    assert local.native_launches == (2 * len(SHAPES) if mode == "per_bucket" else 0)


@pytest.mark.parametrize("kind", ["sgd", "adam", "adam_interleaved"])
def test_explicit_param_buckets_with_two_groups_and_fan_out(gpu, kind):
    """The arenas handed over by the caller (``opt=`` + ``param_buckets=``) instead of built from bucket
    objects: views into one weight arena, one state arena each (or, "adam_interleaved", the moments of all
    buckets in ONE interleaved arena, every bucket naming its first element in it), two parameter groups, one
    replica; through the native meeting point from the second step on."""
    from jabas_amd import sync
    from jabas_amd.local_sync import LocalBucketSync
    interleaved = kind == "adam_interleaved"
    kind = kind.replace("_interleaved", "")
    K, batches, sizes = 2, (3, 1), [70001, 2049]
    opt = _opt_dict("sgd") if kind == "sgd" else dict(kind="adam", betas=(0.9, 0.999), eps=1e-8,
                                                     groups=[dict(lr=2e-3, weight_decay=0.0),
                                                             dict(lr=1e-3, weight_decay=1e-2)])
    total = sum(sizes)
    gen = torch.Generator().manual_seed(9)
    p_h = torch.randn(total, generator=gen) * 0.05
    s1_h, s2_h = torch.zeros(total), torch.zeros(total)
    p_d, s1_d, s2_d, fan = p_h.to(gpu), s1_h.to(gpu), s2_h.to(gpu), torch.zeros(total, device=gpu)
    arena = sync.MomentArena(total, 2, gpu, 10) if interleaved else None
    spans, pbs, off = [], {}, 0
    for b, n in enumerate(sizes):
        bounds = ((0, 0), (n // 3, 1), (2 * n // 3 + 1, 0))
        sl = slice(off, off + n)
        state = dict(moments=(arena, off)) if interleaved else \
            dict(state1=s1_d[sl], state2=None if kind == "sgd" else s2_d[sl])
        pbs[b] = dict(param=p_d[sl], bounds=bounds, fanout=[fan[sl]], **state)
        spans.append((off, n, bounds))
        off += n
    local = LocalBucketSync(batches, opt=opt, param_buckets=pbs)
    bufs = [torch.zeros(total, device=gpu) for _ in range(K)]
    for step in range(1, 4):
        host = [torch.randn(total, generator=torch.Generator().manual_seed(50 * step + k)) * 1e-3 for k in range(K)]
        for k in range(K):
            bufs[k].copy_(host[k])
        for b, (o, n, _) in enumerate(spans):
            for k in (0, 1):                                                    # VSW 0 first
                local.publish(k, b, bufs[k][o:o + n])
        local.finish_step()
        torch.cuda.synchronize()
        agg_h, _ = O.sync_step(host, batches, spans, opt, p_h, s1_h, s2_h, step=step, first_step=(step == 1))
        if interleaved:
            s1_d, s2_d = arena.read(0), arena.read(1)
        assert _same(bufs[0], agg_h) and _same(p_d, p_h) and _same(s1_d, s1_h) and _same(fan, p_h), step
        if kind != "sgd":
            assert _same(s2_d, s2_h), step
    assert local.native_launches == 2 * len(sizes) and local.launched == 3 * len(sizes)


def test_native_meeting_point_errors_and_new_buffers(gpu):
    """Hand-overs of buckets the native meeting point knows: a VSW that never comes, one that comes twice, and
    buffers that change between steps (DDP's bucket rebuild). Every healthy step is bit-exact with the oracle."""
    from jabas_amd.local_sync import LocalBucketSync
    K, batches, sizes = 3, (4, 2, 2), [50001, 4099]
    local = LocalBucketSync(batches)
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]

    def fresh():
        return [[torch.zeros(n, device=gpu) for _ in range(K)] for n in sizes]

    def step(bufs, seed, skip=None, twice=None):
        host = [[torch.randn(n, generator=torch.Generator().manual_seed(seed + 10 * b + k)) * 1e-3 for k in range(K)]
                for b, n in enumerate(sizes)]
        for b in range(len(sizes)):
            for k in (1, 0, 2):                                                  # VSW 0 in the middle
                if (b, k) == skip:
                    continue
                with torch.cuda.stream(streams[k]):
                    bufs[b][k].copy_(host[b][k].to(gpu, non_blocking=False))
                    local.publish(k, b, bufs[b][k])
                    if (b, k) == twice:
                        local.publish(k, b, bufs[b][k])
        return host

    def check(bufs, host):
        torch.cuda.synchronize()
        for b, n in enumerate(sizes):
            agg_h, _ = O.sync_step(host[b], batches, [(0, n, ((0, 0),))], None, None, None, None, step=1, first_step=True)
            assert _same(bufs[b][0], agg_h), b

    bufs = fresh()
    host = step(bufs, 100)                       # described here
    local.finish_step()
    check(bufs, host)
    assert local.native_launches == 0
    host = step(bufs, 200)                       # native
    local.finish_step()
    check(bufs, host)
    assert local.native_launches == len(sizes)
    step(bufs, 300, skip=(1, 2))                 # VSW 2 never hands bucket 1 over
    with pytest.raises(RuntimeError, match="not published by every VSW"):
        local.finish_step()
    host = step(bufs, 400)                       # the next step starts clean
    local.finish_step()
    check(bufs, host)
    step(bufs, 500, twice=(0, 1))                # bucket 0 from VSW 1 twice: reported at the end of the step
    with pytest.raises(RuntimeError):
        local.finish_step()
    local.reset()
    host = step(bufs, 600)
    local.finish_step()
    check(bufs, host)
    before = local.native_launches
    other = fresh()                              # other buffers: described again, native again the step after
    host = step(other, 700)
    local.finish_step()
    check(other, host)
    assert local.native_launches == before
    host = step(other, 800)
    local.finish_step()
    check(other, host)
    assert local.native_launches == before + len(sizes)


@pytest.mark.parametrize("how", ["vsw0_stream", "batched_two_launch_streams", "last_vsw_stream"])
def test_per_bucket_clipping_of_the_gnmt_shard_optimizer(gpu, how):
    """ShardGNMTAdam(grad_clip=) in the hook (examples/gnmt/seq2seq/train/shard_optimizer.py:8-29,75-76):
    every bucket's aggregate is scaled to norm <= grad_clip before Adam sees it. Oracle: the aggregate,
    torch.nn.utils.clip_grad_norm_'s coefficient from its float64 norm, one fp32 product, Adam. Also out of a
    batch of buckets (each bucket still takes launches of its own, on its own launch stream, behind the batch's
    stream waits) and on the stream of the VSW that came last."""
    from jabas_amd import ddp_comm_hooks as H, optim
    from jabas_amd.local_sync import LocalBucketSync
    from jabas_amd.train import create_optimizer_hook
    K, batches = 2, (128, 64)
    shapes = [[(257, 33), (33,)], [(4000,)]]
    gen = torch.Generator().manual_seed(3)
    init = [[torch.randn(s, generator=gen) * 0.05 for s in bucket] for bucket in shapes]
    replicas = [[[torch.nn.Parameter(t.clone().to(gpu)) for t in bucket] for bucket in init] for _ in range(K)]
    layouts = [_layout(bucket) for bucket in shapes]
    bufs = [[torch.zeros(n, device=gpu) for _ in range(K)] for (_, _, n) in layouts]
    clip = 0.05
    optimizer = optim.ShardGNMTAdam([p for bucket in replicas[0] for p in bucket], lr=2e-3, grad_clip=clip)
    opt = dict(kind="adam", betas=(0.9, 0.999), eps=1e-8, groups=[dict(lr=2e-3, weight_decay=0.0)])
    local = LocalBucketSync(batches, **dict(
        vsw0_stream={}, last_vsw_stream=dict(launch_on_last_vsw=True),
        batched_two_launch_streams=dict(stream=torch.cuda.Stream(gpu), launch_streams=2, batch_bytes=1 << 20))[how])
    st = H.IIDPState(None, 2).attach_local(local)
    main_hook = create_optimizer_hook(H.iidp_allreduce_hook, optimizer)
    p_h = [torch.cat([t.reshape(-1) for t in bucket]) for bucket in init]
    s1_h, s2_h = [torch.zeros_like(p) for p in p_h], [torch.zeros_like(p) for p in p_h]
    clipped_any = kept_any = False
    for step in range(1, 4):
        scale = (1e-3, 1e-5, 1e-3)[step - 1]                                   # step 2 stays under the bound
        host = [[torch.randn(n, generator=torch.Generator().manual_seed(77 * step + 5 * b + k)) * scale
                 for k in range(K)] for b, (_, _, n) in enumerate(layouts)]
        for b in range(len(shapes)):
            for k in range(K):
                bufs[b][k].copy_(host[b][k])
                bucket = ParamBucket(b, bufs[b][k], replicas[k][b], layouts[b][0])
                (main_hook(st, bucket) if k == 0 else H.dummy_hook(H.VSWPeerState(local, k), bucket)).wait()
        local.finish_step()
        torch.cuda.synchronize()
        for b, (offs, _, n) in enumerate(layouts):
            agg = O.aggregate(host[b], batches)
            agg, c = O.clip(agg, clip)
            clipped_any, kept_any = clipped_any or c < 1.0, kept_any or c >= 1.0
            O.opt_step(opt, 0, p_h[b], agg, s1_h[b], s2_h[b], step, step == 1)
            assert _same(bufs[b][0], agg), (step, b, "clipped aggregate")
            for i, (p, o) in enumerate(zip(replicas[0][b], offs)):
                assert _same(p.data, p_h[b][o:o + p.numel()]), (step, b, i)
                assert _same(replicas[1][b][i].data, p.data)
    assert clipped_any and kept_any


@pytest.mark.parametrize("amsgrad", [False, True])
def test_shard_gnmt_adam_step_clips_like_clip_grad_norm_then_adam(gpu, amsgrad):
    """ShardGNMTAdam.step(gradients) outside any hook: torch.nn.utils.clip_grad_norm_ over the gradients
    of the call, then torch.optim.Adam, is the library statement of the same step (1e-6; the oracle's
    sequence bit for bit), and the gradient tensors of the call hold the clipped values afterwards."""
    from jabas_amd import optim
    from jabas_amd.train.trainer import tag_parameter_indices
    torch.manual_seed(0)
    model = tag_parameter_indices(torch.nn.Sequential(torch.nn.Linear(40, 50), torch.nn.Linear(50, 7)).to(gpu))
    ref = torch.nn.Sequential(torch.nn.Linear(40, 50), torch.nn.Linear(50, 7)).to(gpu)
    ref.load_state_dict(model.state_dict())
    mine = optim.ShardGNMTAdam(model.parameters(), lr=2e-3, grad_clip=5e-3, amsgrad=amsgrad)
    theirs = torch.optim.Adam(ref.parameters(), lr=2e-3, foreach=False, amsgrad=amsgrad)
    params = list(model.parameters())
    p_h = [p.detach().cpu().clone().reshape(-1) for p in params]
    m_h, v_h = [torch.zeros_like(p) for p in p_h], [torch.zeros_like(p) for p in p_h]
    x_h = [torch.zeros_like(p) if amsgrad else None for p in p_h]
    opt = dict(kind="adam", betas=(0.9, 0.999), eps=1e-8, amsgrad=amsgrad, groups=[dict(lr=2e-3, weight_decay=0.0)])
    flat = torch.zeros(sum(p.numel() for p in params), device=gpu)            # one "bucket"
    for step in range(1, 5):
        scale = (1e-3, 1e-6, 1e-3, 1e-2)[step - 1]                             # step 2 stays under the bound
        host = torch.randn(flat.numel(), generator=torch.Generator().manual_seed(step)) * scale
        flat.copy_(host)
        grads, off = [], 0
        for p, rp in zip(params, ref.parameters()):
            v = flat[off:off + p.numel()].view(p.shape)
            v.index = p.index
            grads.append(v)
            rp.grad = v.detach().clone()
            off += p.numel()
        mine.step(grads)
        torch.nn.utils.clip_grad_norm_(ref.parameters(), 5e-3)
        theirs.step()
        torch.cuda.synchronize()
        clipped, c = O.clip(host, 5e-3)
        assert (c < 1.0) == (step != 2)
        off = 0
        for i, (p, rp) in enumerate(zip(params, ref.parameters())):
            n = p.numel()
            O.opt_step(opt, 0, p_h[i], clipped[off:off + n], m_h[i], v_h[i], step, step == 1, s3=x_h[i])
            off += n
            assert _same(p.data, p_h[i]), (step, i)
            if amsgrad:
                assert _same(mine.state[p]["max_exp_avg_sq"], x_h[i]), (step, i)
            assert torch.allclose(p.data, rp.data, rtol=1e-6, atol=1e-8), (step, i)
        # the gradients handed over are clipped in place, as clip_grad_norm_for_overlap leaves them
        # (examples/gnmt/seq2seq/train/shard_optimizer.py:75-76); untouched when the norm is under the bound
        assert _same(flat, clipped), step
        assert torch.allclose(flat, torch.cat([rp.grad.reshape(-1) for rp in ref.parameters()]), rtol=1e-6, atol=1e-12)
        assert (step == 2) == _same(flat, host)
    with pytest.raises(ValueError, match="param_groups"):
        optim.ShardGNMTAdam([{"params": params[:1]}, {"params": params[1:]}], grad_clip=1.0)


def test_batches_that_would_merge_nothing_fall_back_to_one_launch_per_bucket(gpu):
    """``batch_bytes`` below twice the mean bucket size: a batch would hold one bucket most of the time, so after
    the first step the buckets go out one launch each (and through the native meeting point) again."""
    from jabas_amd.local_sync import LocalBucketSync
    K, batches, sizes = 2, (4, 4), [60000, 50000, 70000]
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    bufs = [[torch.zeros(n, device=gpu) for _ in range(K)] for n in sizes]

    def run(local, steps):
        for step in range(steps):
            host = [[torch.randn(n, generator=torch.Generator().manual_seed(9 * step + 3 * b + k)) * 1e-3
                     for k in range(K)] for b, n in enumerate(sizes)]
            for b in range(len(sizes)):
                for k in range(K):
                    with torch.cuda.stream(streams[k]):
                        bufs[b][k].copy_(host[b][k].to(gpu))
                        local.publish(k, b, bufs[b][k])
            local.finish_step()
            torch.cuda.synchronize()
            for b, n in enumerate(sizes):
                agg_h, _ = O.sync_step(host[b], batches, [(0, n, ((0, 0),))], None, None, None, None, step=1, first_step=True)
                assert _same(bufs[b][0], agg_h), (step, b)

    merging = LocalBucketSync(batches, batch_bytes=600_000)          # 240 kB a bucket: two or three per batch
    run(merging, 3)
    assert merging.batch_bytes == 600_000 and merging.launched < 3 * len(sizes)
    alone = LocalBucketSync(batches, batch_bytes=300_000)            # 1.25 buckets per batch
    run(alone, 4)
    assert alone.batch_bytes == 0
    assert alone.launched > 3 * len(sizes) - 3 and alone.native_launches == 2 * len(sizes)


@pytest.mark.parametrize("interleave", [False, True])
def test_rebuilt_bucket_at_the_old_addresses_is_rebound(gpu, interleave):
    """DDP's bucket rebuild can put the same parameters in another order (or other parameters) at the old buffer
    addresses. With an optimizer bound, the native meeting point must not launch the span it was described for
    the old order: VSW 0's bucket is checked against the parameters of the description, the arenas are laid out
    again, and a peer that had already handed its (unchanged) buffer over natively is handed over again.
    interleave: the moments live in the bucket's interleaved arena and move with their parameter into the new one."""
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    from jabas_amd.train import create_optimizer_hook, create_stream_for_optimizer

    K, batches = 2, (6, 2)
    opt = _opt_dict("adamw")
    shapes = {"vec": (4096,), "mat": (64, 64)}                      # equal sizes, different parameter groups
    gen = torch.Generator().manual_seed(11)
    init = {n: torch.randn(s, generator=gen) * 0.05 for n, s in shapes.items()}
    replicas = [{n: torch.nn.Parameter(t.clone().to(gpu)) for n, t in init.items()} for _ in range(K)]
    optimizer = _torch_optimizer("adamw", list(replicas[0].values()))
    local = LocalBucketSync(batches, stream=create_stream_for_optimizer(gpu), interleave_moments=interleave)
    st = H.GradientSimilarityState(None, 2, None, [], 10 ** 9).attach_local(local)
    main_hook = create_optimizer_hook(H.similimarity_allreduce_hook(H.subgroup_allreduce_hook), optimizer)
    bufs = [torch.zeros(8192, device=gpu) for _ in range(K)]
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    p_h = {n: t.clone().reshape(-1) for n, t in init.items()}
    s1_h = {n: torch.zeros(4096) for n in shapes}
    s2_h = {n: torch.zeros(4096) for n in shapes}
    group = {"vec": 0, "mat": 1}
    # (order of the parameters in the bucket, who hands over first)
    plan = [(("vec", "mat"), 0), (("vec", "mat"), 1), (("mat", "vec"), 0), (("mat", "vec"), 1), (("vec", "mat"), 1),
            (("vec", "mat"), 0)]
    native_before = 0
    for step, (order, first) in enumerate(plan, start=1):
        host = [torch.randn(8192, generator=torch.Generator().manual_seed(50 * step + k)) * 1e-3 for k in range(K)]
        for k in ([0, 1] if first == 0 else [1, 0]):
            with torch.cuda.stream(streams[k]):
                bufs[k].copy_(host[k].to(gpu))
                bucket = ParamBucket(0, bufs[k], [replicas[k][n] for n in order], [0, 4096])
                if k == 0:
                    main_hook(st, bucket).wait()
                else:
                    H.dummy_hook(H.VSWPeerState(local, k), bucket).wait()
        local.finish_step()
        torch.cuda.synchronize()
        seen = _checkpointed(optimizer) if interleave else {id(p): optimizer.state[p] for p in replicas[0].values()}
        for j, n in enumerate(order):
            sl = slice(4096 * j, 4096 * (j + 1))
            agg = O.aggregate([host[k][sl] for k in range(K)], batches)
            O.opt_step(opt, group[n], p_h[n], agg, s1_h[n], s2_h[n], step, step == 1)
            assert _same(bufs[0][sl], agg), (step, n, "aggregate")
            assert _same(replicas[0][n].data, p_h[n]), (step, n, "weights")
            assert _same(replicas[1][n].data, p_h[n]), (step, n, "replica")
            assert _same(seen[id(replicas[0][n])]["exp_avg"], s1_h[n]), (step, n)
            assert _same(seen[id(replicas[0][n])]["exp_avg_sq"], s2_h[n]), (step, n)
            assert ("exp_avg" in optimizer.state[replicas[0][n]]) == (not interleave)
        # natively launched: a step whose bucket came as the step before left it
        want_native = step >= 2 and plan[step - 2][0] == order
        assert local.native_launches - native_before == (1 if want_native else 0), step
        native_before = local.native_launches
        st.step += 1


def test_statistics_rows_keep_alternating_when_a_bucket_moves_to_the_native_meeting_point(gpu):
    """A bucket's statistics launches alternate between two device rows, so that the row a step handed out stays
    valid until the second-next statistics step. The first launch of a bucket goes through the Python path, the
    following ones through the native meeting point: the alternation continues across the two."""
    from jabas_amd.local_sync import LocalBucketSync
    K, batches, n = 2, (3, 1), 40_001
    local = LocalBucketSync(batches)
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    bufs = [torch.zeros(n, device=gpu) for _ in range(K)]
    handed, want = [], []

    for step in range(4):
        host = [torch.randn(n, generator=torch.Generator().manual_seed(77 * step + k)) * 1e-3 for k in range(K)]
        want.append(O.stats(host, batches))
        for k in (1, 0):
            with torch.cuda.stream(streams[k]):
                bufs[k].copy_(host[k].to(gpu))
                local.publish(k, 0, bufs[k], want_stats=True, on_done=handed.append if k == 0 else None)
        local.finish_step()
        torch.cuda.synchronize()
        assert local.native_launches == step                      # the first launch describes the bucket, the rest are native
        assert len(handed) == step + 1
        # this step's row and the one before it are both intact; the one before that has been written over
        for back in (0, 1):
            if step - back >= 0:
                got = handed[step - back].cpu()
                assert torch.allclose(got[1:4], want[step - back][1:4], rtol=1e-6, atol=0.0), (step, back)
        if step >= 2:
            assert handed[step].row.data_ptr() == handed[step - 2].row.data_ptr()
            assert handed[step].row.data_ptr() != handed[step - 1].row.data_ptr()


@pytest.mark.parametrize("kind,interleave", [("sgd", False), ("adamw", False), ("adamw", True), ("adamw_amsgrad", True)])
def test_optimizer_load_state_dict_after_the_buckets_are_bound(gpu, kind, interleave):
    """``optimizer.load_state_dict`` replaces the tensors in ``optimizer.state``; the launches read the arenas.
    Two steps, a checkpoint (weights + ``optimizer.state_dict()``), two more steps, then the checkpoint is loaded
    back and steps 3 and 4 are taken again: weights and state must be the oracle's after four steps, bit for bit
    (a launch that kept using what its arenas held would apply steps 5 and 6 to them)."""
    import copy
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    from jabas_amd.train import create_optimizer_hook
    K, batches, shapes = 2, (6, 2), SHAPES[:2]
    opt = _opt_dict(kind)
    gen = torch.Generator().manual_seed(11)
    init = [[torch.randn(s, generator=gen) * 0.05 for s in bucket] for bucket in shapes]
    replicas = [[[torch.nn.Parameter(t.clone().to(gpu)) for t in bucket] for bucket in init] for _ in range(K)]
    layouts = [_layout(bucket) for bucket in shapes]
    bufs = [[torch.zeros(n, device=gpu) for _ in range(K)] for (_, _, n) in layouts]
    optimizer = _torch_optimizer(kind, [p for bucket in replicas[0] for p in bucket])
    local = LocalBucketSync(batches, interleave_moments=interleave)
    st = H.IIDPState(None, 2).attach_local(local)
    main_hook = create_optimizer_hook(H.iidp_allreduce_hook, optimizer)
    host = {step: [[torch.randn(n, generator=torch.Generator().manual_seed(31 * step + 7 * b + k)) * 1e-3
                    for k in range(K)] for b, (_, _, n) in enumerate(layouts)] for step in range(1, 5)}

    def take(step):
        for b in range(len(shapes)):
            for k in range(K):
                bufs[b][k].copy_(host[step][b][k])
                bucket = ParamBucket(b, bufs[b][k], replicas[k][b], layouts[b][0])
                (main_hook(st, bucket) if k == 0 else H.dummy_hook(H.VSWPeerState(local, k), bucket)).wait()
        local.finish_step()

    take(1)
    take(2)
    torch.cuda.synchronize()
    saved_w = [[p.detach().clone() for p in bucket] for bucket in replicas[0]]
    saved_o = copy.deepcopy(optimizer.state_dict())
    take(3)
    take(4)
    torch.cuda.synchronize()
    with torch.no_grad():
        for model in replicas:
            for bucket, saved in zip(model, saved_w):
                for p, w in zip(bucket, saved):
                    p.copy_(w)                                                  # in place: the views stay
    optimizer.load_state_dict(saved_o)
    assert kind == "sgd" or local.step_count == 2            # Adam's t follows the checkpoint; SGD keeps no count
    take(3)
    take(4)
    torch.cuda.synchronize()
    seen = _checkpointed(optimizer)
    for b, (offs, bounds, n) in enumerate(layouts):
        p_h = torch.cat([t.reshape(-1) for t in init[b]])
        s1_h, s2_h = torch.zeros_like(p_h), torch.zeros_like(p_h)
        s3_h = torch.zeros_like(p_h) if kind.endswith("amsgrad") else None
        for step in range(1, 5):
            O.sync_step(host[step][b], batches, [(0, n, bounds)], opt, p_h, s1_h, s2_h, step=step,
                        first_step=(step == 1), want_stats=False, state3=s3_h)
        for i, (p, o) in enumerate(zip(replicas[0][b], offs)):
            sl = slice(o, o + p.numel())
            assert _same(p.data, p_h[sl]), (b, i, "weights")
            assert _same(replicas[1][b][i].data, p.data), (b, i, "replica")
            state = seen[id(p)]
            if kind == "sgd":
                assert _same(state["momentum_buffer"], s1_h[sl]), (b, i, "momentum")
            else:
                assert int(state["step"]) == 4
                assert _same(state["exp_avg"], s1_h[sl]) and _same(state["exp_avg_sq"], s2_h[sl]), (b, i, "moments")
                if s3_h is not None:
                    assert _same(state["max_exp_avg_sq"], s3_h[sl]), (b, i, "maximum")
