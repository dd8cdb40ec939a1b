"""GPU tests of the flat-arena engine: multi-bucket plans with parameter groups, in-place
aggregation, fan-out, per-tensor spans, and global-norm clipping (two launches with a
device-side coefficient), against the oracle over the same arenas."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

from jabas_amd import _lib as L

from oracle import oracle as O
from jabas_amd.workloads import ParamSpec

pytestmark = pytest.mark.gpu

SPECS = [ParamSpec("a.weight", 5000, 1), ParamSpec("a.bias", 77, 0), ParamSpec("b.weight", 300000, 1),
         ParamSpec("b.bias", 1024, 0), ParamSpec("c.weight", 64 * 64 * 9, 1), ParamSpec("c.scale", 1, 0),
         ParamSpec("d.weight", 123457, 1)]
CAPS = (4096 * 4, 200000 * 4)
SGD = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
           groups=[dict(lr=0.1, weight_decay=0.0), dict(lr=0.1, weight_decay=1e-4)])
ADAM = dict(kind="adam", betas=(0.9, 0.999), eps=1e-8,
            groups=[dict(lr=2e-3, weight_decay=0.0), dict(lr=2e-3, weight_decay=1e-2)])


def _close(a, b, rtol=1e-6, atol=1e-9):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    return bool(((a - b).abs() <= rtol * b.abs() + atol).all())


def _make(gpu, batches, opt, dtype=torch.float32, **kw):
    from jabas_amd.engine import VSWFlatSync
    eng = VSWFlatSync(SPECS, batches, grad_dtype=dtype, opt=opt, device=gpu, caps=CAPS, **kw)
    gen = torch.Generator().manual_seed(3)
    n = eng.layout.total
    host = dict(g=[(torch.randn(n, generator=gen) * 1e-2).to(dtype) for _ in batches],
                p=torch.randn(n, generator=gen) * 0.05, s1=torch.zeros(n), s2=torch.zeros(n))
    for k, g in enumerate(host["g"]):
        eng.grads[k].copy_(g)
    eng.param.copy_(host["p"])
    spans = [(off, cnt, bounds) for off, cnt, bounds, _ in eng.layout.spans]
    return eng, host, spans


@pytest.mark.parametrize("per_tensor", [False, True])
@pytest.mark.parametrize("opt,dtype,blocks", [(SGD, torch.float32, 13), (ADAM, torch.float32, 13), (ADAM, torch.bfloat16, 13),
                                              (ADAM, torch.float32, 0), (ADAM, torch.bfloat16, 9)])
def test_engine_steps_match_oracle(gpu, opt, dtype, per_tensor, blocks):
    """blocks: log2 of the block size of the interleaved moment arena (the engine's default 13; 9: blocks smaller
    than a tile; 0: flat state arenas)."""
    batches = (4, 2, 2)
    eng, host, spans = _make(gpu, batches, opt, dtype, n_fanout=2, per_tensor_spans=per_tensor, moment_block_log2=blocks)
    assert eng.state_is_live == (opt is SGD or blocks == 0)
    assert len(eng.layout.buckets) >= 3
    adam = opt["kind"] != "sgd"
    for step in (1, 2, 3):
        rows = eng.step(stats=True)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(host["g"], batches, spans, opt, host["p"], host["s1"], host["s2"] if adam else None,
                                    step=step, first_step=(step == 1), want_stats=True)
        for off, cnt, _ in spans:
            sl = slice(off, off + cnt)
            assert torch.equal(eng.agg[sl].cpu().view(torch.int32), agg_h[sl].view(torch.int32)), step
        rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
        assert _close(rows[:, :7], rows_h[:, :7], rtol, 1e-30)
        assert _close(eng.param, host["p"]) and _close(eng.state1, host["s1"], 1e-6, 2e-9)
        for f in eng.fanout:
            for off, cnt, _ in spans:                             # padding between buckets is never touched
                assert torch.equal(f[off:off + cnt], eng.param[off:off + cnt])
        assert eng.cosine(rows) == pytest.approx(O.cosine_from_rows(rows_h), rel=1e-6)
        if dtype == torch.float32:
            for off, cnt, _ in spans:
                host["g"][0][off:off + cnt] = agg_h[off:off + cnt]
        per_bucket = eng.bucket_stats(rows)
        assert per_bucket.shape[0] == len(eng.layout.buckets)
        assert torch.allclose(per_bucket.sum(0), rows.cpu().sum(0), rtol=1e-12)


@pytest.mark.parametrize("clip_norm,keep", [(0.05, True), (1e3, True), (0.05, False)])
@pytest.mark.parametrize("opt", [SGD, ADAM])
def test_global_norm_clipping(gpu, opt, clip_norm, keep):
    batches = (128, 128, 64, 64)
    eng, host, spans = _make(gpu, batches, opt, n_fanout=1, keep_clipped_grads=keep)
    adam = opt["kind"] != "sgd"
    for step in (1, 2):
        rows = eng.step(stats=True, clip_norm=clip_norm)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(host["g"], batches, spans, opt, host["p"], host["s1"], host["s2"] if adam else None,
                                    step=step, first_step=(step == 1), want_stats=True, clip_norm=clip_norm)
        total = float(rows_h[:, O.NORM_AGG].sum())
        c = O.clip_coef(total, clip_norm)
        assert (c < 1.0) == (clip_norm < 1.0)                     # the small bound clips, the large one does not
        assert float(eng._coef) == pytest.approx(c, rel=1e-6)
        assert _close(rows[:, :8], rows_h[:, :8], 1e-6, 1e-30)     # statistics are of the unclipped aggregate
        for off, cnt, _ in spans:
            sl = slice(off, off + cnt)
            if keep:
                assert _close(eng.agg[sl], agg_h[sl], 1e-6, 1e-12), step
            else:                                                  # the unclipped aggregate stays behind
                assert _close(eng.agg[sl] * c, agg_h[sl], 1e-6, 1e-12), step
            if c >= 1.0:
                assert torch.equal(eng.agg[sl].cpu().view(torch.int32), agg_h[sl].view(torch.int32))
        assert _close(eng.param, host["p"]) and _close(eng.state1, host["s1"], 1e-6, 2e-9)
        for off, cnt, _ in spans:
            assert torch.equal(eng.fanout[0][off:off + cnt], eng.param[off:off + cnt])
            # the in-place aggregate is worker 0's input of the next step
            host["g"][0][off:off + cnt] = agg_h[off:off + cnt] if keep else eng.agg[off:off + cnt].cpu()
    if clip_norm < 1.0 and keep:
        norm = math.sqrt(sum(float(torch.dot(eng.agg[o:o + c_].double(), eng.agg[o:o + c_].double())) for o, c_, _ in spans))
        assert norm == pytest.approx(clip_norm, rel=1e-4)


@pytest.mark.parametrize("opt,dtype,batches", [(SGD, torch.float32, (4, 2, 1, 1)), (ADAM, torch.bfloat16, (4, 2, 1, 1)),
                                               (ADAM, torch.bfloat16, (64, 56, 48, 40, 32, 24, 16, 8)),
                                               (ADAM, torch.float32, (7, 7, 5, 3, 2, 1))])
@pytest.mark.parametrize("clip", [None, 0.05])
def test_engine_gram_rows_out_of_the_step(gpu, opt, dtype, batches, clip):
    """stats="gram": the planned launch over every span leaves the pair products beside the full rows (with
    clipping: the aggregate launch does), and the step itself stays what it is without them. Four workers, and
    the eight bf16 ones of the largest configuration."""
    K = len(batches)
    eng, host, spans = _make(gpu, batches, opt, dtype, per_tensor_spans=True)
    plain, host2, _ = _make(gpu, batches, opt, dtype, per_tensor_spans=True)
    for step in (1, 2):
        for k, g in enumerate(host["g"]):       # fp32 engines aggregate into VSW 0's arena: the same inputs every step
            eng.grads[k].copy_(g)
            plain.grads[k].copy_(g)
        rows = eng.step(stats="gram", clip_norm=clip)
        plain.step(stats=False, clip_norm=clip)
        torch.cuda.synchronize()
        assert rows.shape == (len(spans), L.STATS_STRIDE)
        assert torch.count_nonzero(rows[:, 4 + K + K * (K - 1) // 2:]) == 0
        want = O.gram([torch.cat([g[o:o + n] for o, n, _ in spans]) for g in host["g"]])
        scale = torch.sqrt(torch.outer(torch.diagonal(want), torch.diagonal(want)))
        tol = 1e-11 if dtype == torch.float32 else 1e-5
        assert bool(((eng.gram(rows).cpu() - want).abs() <= tol * scale).all())
        rows_h = torch.stack([O.stats([g[o:o + n] for g in host["g"]], batches) for o, n, _ in spans])
        assert _close(rows[:, 1:4 + K], rows_h[:, 1:4 + K], tol, 1e-30)
        assert torch.equal(eng.param.view(torch.int32), plain.param.view(torch.int32))
        assert torch.equal(eng.state1.view(torch.int32), plain.state1.view(torch.int32))


@pytest.mark.parametrize("dtype,clip", [(torch.float32, None), (torch.bfloat16, None), (torch.float32, 0.05)])
def test_engine_amsgrad_matches_oracle(gpu, dtype, clip):
    """A planned launch over several buckets and parameter groups with amsgrad, plain and under a global norm
    bound: weights, both moments and the maximum bit-identical to the oracle; an amsgrad step is not recordable."""
    batches = (4, 2, 2)
    opt = dict(ADAM, amsgrad=True)
    eng, host, spans = _make(gpu, batches, opt, dtype, n_fanout=1)
    host["s3"] = torch.zeros(eng.layout.total)
    assert eng.state3 is not None
    for step in (1, 2, 3, 4):
        gen = torch.Generator().manual_seed(900 + step)
        host["g"] = [(torch.randn(eng.layout.total, generator=gen) * (5e-2 if step <= 2 else 2e-3)).to(dtype) for _ in batches]
        for k, g in enumerate(host["g"]):
            eng.grads[k].copy_(g)
        eng.step(stats="similarity", clip_norm=clip)
        torch.cuda.synchronize()
        O.sync_step(host["g"], batches, spans, opt, host["p"], host["s1"], host["s2"], step=step, want_stats=False,
                    clip_norm=clip, state3=host["s3"])
        for off, cnt, _ in spans:
            sl = slice(off, off + cnt)
            for name, d, h in (("p", eng.param, host["p"]), ("m", eng.state1, host["s1"]), ("v", eng.state2, host["s2"]),
                               ("max", eng.state3, host["s3"]), ("replica", eng.fanout[0], host["p"])):
                assert torch.equal(d[sl].cpu().view(torch.int32), h[sl].view(torch.int32)), (step, name)
    with pytest.raises(ValueError, match="amsgrad"):
        eng.capture()


def test_reconfigure_changes_k_and_keeps_weights_and_state(gpu):
    batches = (4, 4)
    eng, host, spans = _make(gpu, batches, ADAM, n_fanout=1)
    eng.step()
    O.sync_step(host["g"], batches, spans, ADAM, host["p"], host["s1"], host["s2"], step=1, first_step=True)
    torch.cuda.synchronize()
    p_before, m_before = eng.param.clone(), eng.state1.clone()
    # grow to 3 workers, shrink to 1, grow past 8, to the maximum, and back
    for new_batches, step in (((4, 4, 4), 2), ((4,), 3), ((2,) * 11, 4), (tuple(range(16, 0, -1)), 5), ((8, 8), 6)):
        eng.reconfigure(new_batches)
        assert eng.K == len(new_batches) and len(eng.grads) == eng.K and len(eng.fanout) == eng.K - 1
        assert torch.equal(eng.param, p_before) and torch.equal(eng.state1, m_before)
        assert eng.step_count == step - 1
        for f in eng.fanout:
            for off, cnt, _ in spans:
                assert torch.equal(f[off:off + cnt], eng.param[off:off + cnt])     # a new replica starts in sync
        gen = torch.Generator().manual_seed(40 + step)
        hg = [torch.randn(eng.layout.total, generator=gen) * 1e-2 for _ in new_batches]
        for k, g in enumerate(hg):
            eng.grads[k].copy_(g)
        rows = eng.step(stats=True)
        torch.cuda.synchronize()
        agg_h, rows_h = O.sync_step(hg, new_batches, spans, ADAM, host["p"], host["s1"], host["s2"], step=step,
                                    first_step=False, want_stats=True)
        for off, cnt, _ in spans:
            assert torch.equal(eng.agg[off:off + cnt].cpu().view(torch.int32), agg_h[off:off + cnt].view(torch.int32))
        assert _close(eng.param, host["p"]) and _close(eng.state1, host["s1"], 1e-6, 2e-9)
        assert _close(rows[:, :4 + eng.K], rows_h[:, :4 + eng.K], 1e-6, 1e-30)
        p_before, m_before = eng.param.clone(), eng.state1.clone()


@pytest.mark.parametrize("opt", [SGD, ADAM])
def test_lr_modifier_that_moves_between_steps_is_bit_exact(gpu, opt):
    """The adaptive-batching LR modifier (jabas/train/trainer.py:693-700: lr *= modifier before the
    step, /= after) travels as ``lr_scale`` of the launch: weights and state bit for bit against the
    oracle stepping at lr * modifier, with the modifier changing from step to step."""
    batches = (48, 32, 32, 16)
    eng, host, spans = _make(gpu, batches, opt, n_fanout=1)
    adam = opt["kind"] != "sgd"
    mods = (1.0, math.sqrt(20 / 8), math.sqrt(20 / 8), 0.5, 1.0 / 3.0)
    for step, m in enumerate(mods, 1):
        gen = torch.Generator().manual_seed(90 + step)
        for k in range(len(batches)):
            host["g"][k] = torch.randn(eng.layout.total, generator=gen) * 1e-2
            eng.grads[k].copy_(host["g"][k])
        eng.step(lr_scale=m)
        torch.cuda.synchronize()
        O.sync_step(host["g"], batches, spans, opt, host["p"], host["s1"], host["s2"] if adam else None, step=step,
                    first_step=(step == 1), lr_scale=m)
        for off, cnt, _ in spans:
            sl = slice(off, off + cnt)
            assert torch.equal(eng.param[sl].cpu().view(torch.int32), host["p"][sl].view(torch.int32)), (step, m)
            assert torch.equal(eng.state1[sl].cpu().view(torch.int32), host["s1"][sl].view(torch.int32)), (step, m)
            if adam:
                assert torch.equal(eng.state2[sl].cpu().view(torch.int32), host["s2"][sl].view(torch.int32)), (step, m)
            assert torch.equal(eng.fanout[0][sl], eng.param[sl])
    # the modifier did change the trajectory: the same steps at modifier 1 end elsewhere
    eng2, host2, _ = _make(gpu, batches, opt)
    for step in range(1, len(mods) + 1):
        gen = torch.Generator().manual_seed(90 + step)
        for k in range(len(batches)):
            eng2.grads[k].copy_(torch.randn(eng2.layout.total, generator=gen) * 1e-2)
        eng2.step()
    assert not torch.equal(eng2.param, eng.param)


@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_parameter_groups_at_different_adam_step_counts(gpu, kind):
    """Groups whose parameters were stepped apart (a group added later, Shard* steps over some buckets
    only) carry their own step count: bias corrections per group, bit for bit against the oracle."""
    from jabas_amd import sync
    n, K, batches = 200_003, 2, (3, 1)
    bounds = ((0, 0), (70_001, 1), (150_002, 0))
    gen = torch.Generator().manual_seed(11)
    p_h = torch.randn(n, generator=gen) * 0.05
    m_h, v_h = torch.randn(n, generator=gen) * 1e-3, torch.rand(n, generator=gen) * 1e-6
    p_d, m_d, v_d = p_h.to(gpu), m_h.to(gpu), v_h.to(gpu)
    steps = [3, 7]
    for it in range(3):
        opt = dict(kind=kind, betas=(0.9, 0.999), eps=1e-8,
                   groups=[dict(lr=1e-3, weight_decay=0.01, step=steps[0] + it),
                           dict(lr=2e-3, weight_decay=0.0, step=steps[1] + it)])
        hg = [torch.randn(n, generator=gen) * 1e-3 for _ in range(K)]
        dg = [g.to(gpu) for g in hg]
        span = sync.SpanSpec(dg, agg_out=dg[0], param=p_d, state1=m_d, state2=v_d, bounds=bounds)
        args = sync.make_step_args(batches, torch.float32, opt=opt, step=1)
        assert [args.groups[i].step for i in range(2)] == [steps[0] + it, steps[1] + it]
        sync.sync_bucket(span, args)
        torch.cuda.synchronize()
        O.sync_step(hg, batches, [(0, n, bounds)], opt, p_h, m_h, v_h, step=1)
        for got, want in ((p_d, p_h), (m_d, m_h), (v_d, v_h)):
            assert torch.equal(got.cpu().view(torch.int32), want.view(torch.int32)), it
    # one common step count gives other weights: the per-group counts were used
    q_h = p_h.clone()
    O.sync_step(hg, batches, [(0, n, bounds)], dict(opt, groups=[dict(g, step=5) for g in opt["groups"]]), q_h,
                m_h.clone(), v_h.clone(), step=1)
    assert not torch.equal(q_h, p_h)


ADAMW = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
             groups=[dict(lr=5e-4, weight_decay=0.0), dict(lr=5e-4, weight_decay=0.05)])


@pytest.mark.parametrize("opt,dtype,batches,stats", [
    (ADAMW, torch.float32, (48, 32, 32, 16), "similarity"),
    (ADAM, torch.bfloat16, (64, 56, 48, 40, 32, 24, 16, 8), "similarity"),
    (ADAM, torch.float32, (3, 2, 1), True),
    (SGD, torch.float32, (4, 2, 2), False),
    (SGD, torch.bfloat16, (2,) * 9, True),
    (ADAMW, torch.bfloat16, (5, 3, 2, 2), "gram"),
])
def test_recorded_step_replays_with_the_scalars_of_the_moment(gpu, opt, dtype, batches, stats):
    """A step recorded ONCE in a HIP graph, replayed from the very first step on (SGD's first-step flag, Adam's
    bias corrections and an LR modifier that changes every step all reach the recorded launch through the
    step-scalar block in device memory): aggregate, weights and optimizer state bit for bit against the oracle
    at every replay, with fresh gradients, eager work and synchronisations between the replays, and bit for
    bit against the same steps launched one by one."""
    K = len(batches)
    eng, host, spans = _make(gpu, batches, opt, dtype, n_fanout=1)
    eager, _, _ = _make(gpu, batches, opt, dtype)
    adam = opt["kind"] != "sgd"
    graphed = eng.capture(stats=stats)
    mods = (1.0, math.sqrt(20 / 8), 0.5, 1.0 / 3.0, 1.0)
    for step, m in enumerate(mods, 1):
        gen = torch.Generator().manual_seed(500 + step)
        for k in range(K):
            host["g"][k] = (torch.randn(eng.layout.total, generator=gen) * 1e-2).to(dtype)
            eng.grads[k].copy_(host["g"][k])
            eager.grads[k].copy_(host["g"][k])
        scratch = (eng.grads[K - 1].float() * 2.0).sum()           # a library reduction between the replays
        rows = graphed.replay(lr_scale=m)
        rows_e = eager.step(stats=stats, lr_scale=m)
        torch.cuda.synchronize()
        assert torch.isfinite(scratch) and eng.step_count == step
        # the block on the device holds what the host encoder gives for this step's arguments
        eng.step_count -= 1
        block = np.zeros(L.STEP_SCALARS_BYTES, dtype=np.uint8)
        L.check(L.lib().jabas_step_scalars_encode(C.byref(eng.step_args(stats=stats, lr_scale=m)), block.ctypes.data,
                                                  block.nbytes), "encode")
        eng.step_count += 1
        assert np.array_equal(graphed.scalars.dev.cpu().numpy(), block)
        agg_h, rows_h = O.sync_step(host["g"], batches, spans, opt, host["p"], host["s1"], host["s2"] if adam else None,
                                    step=step, first_step=(step == 1), want_stats=bool(stats), lr_scale=m)
        for off, cnt, _ in spans:
            sl = slice(off, off + cnt)
            assert torch.equal(eng.agg[sl].cpu().view(torch.int32), agg_h[sl].view(torch.int32)), (step, m)
            assert torch.equal(eng.param[sl].cpu().view(torch.int32), host["p"][sl].view(torch.int32)), (step, m)
            assert torch.equal(eng.state1[sl].cpu().view(torch.int32), host["s1"][sl].view(torch.int32)), (step, m)
            if adam:
                assert torch.equal(eng.state2[sl].cpu().view(torch.int32), host["s2"][sl].view(torch.int32)), (step, m)
            assert torch.equal(eng.fanout[0][sl], eng.param[sl])
            assert torch.equal(eager.param[sl], eng.param[sl])
        if stats:
            assert torch.equal(rows, rows_e)                       # same kernels' arithmetic, same order
            rtol = 1e-2 if dtype == torch.bfloat16 else 1e-6
            width = 4 if stats == "similarity" else 4 + K
            assert _close(rows[:, :width], rows_h[:, :width], rtol, 1e-30)
            if stats == "gram":                                    # the recorded launch leaves the pair products too
                want = O.gram([torch.cat([g[o:o + n] for o, n, _ in spans]) for g in host["g"]])
                scale = torch.sqrt(torch.outer(torch.diagonal(want), torch.diagonal(want)))
                assert bool(((eng.gram(rows).cpu() - want).abs() <= 1e-5 * scale).all())


def test_recorded_clipped_step_and_reconfigure(gpu):
    """Global-norm clipping inside the recording (aggregate + sums, coefficient on the device, Adam over the
    scaled aggregate: three launches, one graph), three replays against the oracle; a recording made before
    ``reconfigure`` refuses to replay."""
    batches = (128, 128, 64, 64)
    eng, host, spans = _make(gpu, batches, ADAM, n_fanout=1)
    graphed = eng.capture(clip_norm=0.05)
    for step in (1, 2, 3):
        gen = torch.Generator().manual_seed(700 + step)
        for k in range(len(batches)):
            host["g"][k] = torch.randn(eng.layout.total, generator=gen) * 1e-2
            eng.grads[k].copy_(host["g"][k])
        graphed.replay(lr_scale=1.0 + 0.25 * step)
        torch.cuda.synchronize()
        O.sync_step(host["g"], batches, spans, ADAM, host["p"], host["s1"], host["s2"], step=step,
                    first_step=(step == 1), lr_scale=1.0 + 0.25 * step, clip_norm=0.05)
        assert float(eng._coef) < 1.0
        assert _close(eng.param, host["p"]) and _close(eng.state1, host["s1"], 1e-6, 2e-9)
        assert _close(eng.state2, host["s2"], 1e-6, 1e-12)
    eng.reconfigure((4, 4))
    with pytest.raises(RuntimeError, match="record it again"):
        graphed.replay()


@pytest.mark.parametrize("opt,dtype", [(SGD, torch.float32), (ADAM, torch.bfloat16)])
def test_step_that_writes_no_aggregate(gpu, opt, dtype):
    """``write_aggregate=False`` (the trainer's setting: it clears the buckets right after the step): weights,
    state, replicas and statistics bit for bit those of the step that writes the aggregate; the gradient buckets
    are left exactly as backward filled them; no aggregate arena exists until a clipped step needs one."""
    batches = (4, 2, 2)
    eng, host, spans = _make(gpu, batches, opt, dtype, n_fanout=1, write_aggregate=False)
    ref, _, _ = _make(gpu, batches, opt, dtype, n_fanout=1)
    assert eng.agg is (eng.grads[0] if dtype == torch.float32 else None)
    adam = opt["kind"] != "sgd"
    for step in (1, 2, 3):
        gen = torch.Generator().manual_seed(800 + step)
        for k in range(len(batches)):
            host["g"][k] = (torch.randn(eng.layout.total, generator=gen) * 1e-2).to(dtype)
            eng.grads[k].copy_(host["g"][k])
            ref.grads[k].copy_(host["g"][k])
        rows = eng.step(stats="similarity")
        rows_ref = ref.step(stats="similarity")
        torch.cuda.synchronize()
        O.sync_step(host["g"], batches, spans, opt, host["p"], host["s1"], host["s2"] if adam else None, step=step,
                    first_step=(step == 1))
        assert torch.equal(rows, rows_ref)
        for off, cnt, _ in spans:
            sl = slice(off, off + cnt)
            assert torch.equal(eng.param[sl].cpu().view(torch.int32), host["p"][sl].view(torch.int32)), step
            assert torch.equal(eng.param[sl], ref.param[sl]) and torch.equal(eng.state1[sl], ref.state1[sl])
            assert torch.equal(eng.fanout[0][sl], eng.param[sl])
        for k in range(len(batches)):                              # every bucket as it was handed in, VSW 0's included
            assert torch.equal(eng.grads[k].cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                               host["g"][k].view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    # a clipped step passes the aggregate from its first launch to its second: the arena appears then
    for k in range(len(batches)):                                  # (the other engine's VSW 0 bucket holds its aggregate by now)
        ref.grads[k].copy_(host["g"][k])
    eng.step(clip_norm=0.05)
    ref.step(clip_norm=0.05)
    torch.cuda.synchronize()
    assert eng.agg is not None
    for off, cnt, _ in spans:
        assert torch.equal(eng.param[off:off + cnt], ref.param[off:off + cnt])
