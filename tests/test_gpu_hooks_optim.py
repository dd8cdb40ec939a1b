"""GPU tests of the host layer above the C ABI: Shard optimizers against torch.optim,
the K-VSW rendezvous with real streams and threads against the oracle, and the slim
trainer end to end against a plain-torch restatement of one training step.
Tolerances: weights 1e-6 relative (absolute floor of a few ulp of the operands),
aggregate bit-exact, statistics 1e-6 relative.
"""
import copy
import threading

import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _close(a, b, rtol=1e-6, atol=1e-9):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    return bool(((a - b).abs() <= rtol * b.abs() + atol).all())


def _mlp(seed):
    torch.manual_seed(seed)
    return torch.nn.Sequential(torch.nn.Linear(37, 64), torch.nn.ReLU(), torch.nn.Linear(64, 33, bias=True),
                               torch.nn.ReLU(), torch.nn.Linear(33, 10))


def _states(opt):
    """id(parameter) -> its entry of ``opt.state_dict()["state"]``: what a checkpoint sees."""
    sd = opt.state_dict()
    params = [p for g in opt.param_groups for p in g["params"]]
    index = [i for g in sd["param_groups"] for i in g["params"]]
    return {id(p): sd["state"][i] for p, i in zip(params, index) if i in sd["state"]}


def _groups(model):
    decay = [p for p in model.parameters() if p.dim() > 1]
    no_decay = [p for p in model.parameters() if p.dim() <= 1]
    return [{"params": no_decay, "weight_decay": 0.0}, {"params": decay, "weight_decay": 0.05}]


@pytest.mark.parametrize("kind", ["sgd", "sgd_nesterov", "adam", "adamw", "adam_amsgrad", "adamw_amsgrad", "gnmt_adam_amsgrad"])
def test_shard_optimizers_match_torch_optim(gpu, kind):
    from jabas_amd import optim
    ref_model, my_model = _mlp(0).to(gpu), _mlp(0).to(gpu)
    if kind == "sgd":
        ref = torch.optim.SGD(_groups(ref_model), lr=0.1, momentum=0.9, foreach=False)
        mine = optim.ShardSGD(_groups(my_model), lr=0.1, momentum=0.9)
    elif kind == "sgd_nesterov":
        ref = torch.optim.SGD(_groups(ref_model), lr=0.05, momentum=0.8, nesterov=True, foreach=False)
        mine = optim.ShardSGD(_groups(my_model), lr=0.05, momentum=0.8, nesterov=True)
    elif kind == "adam":
        ref = torch.optim.Adam(_groups(ref_model), lr=2e-3, foreach=False)
        mine = optim.ShardAdam(_groups(my_model), lr=2e-3)
    elif kind == "adam_amsgrad":
        ref = torch.optim.Adam(_groups(ref_model), lr=2e-3, foreach=False, amsgrad=True)
        mine = optim.ShardAdam(_groups(my_model), lr=2e-3, amsgrad=True)
    elif kind == "adamw_amsgrad":
        ref = torch.optim.AdamW(_groups(ref_model), lr=5e-4, foreach=False, amsgrad=True)
        mine = optim.ShardAdamW(_groups(my_model), lr=5e-4, amsgrad=True)
    elif kind == "gnmt_adam_amsgrad":           # the reference's own subclass, amsgrad threaded through as it does
        ref = torch.optim.Adam(ref_model.parameters(), lr=2e-3, foreach=False, amsgrad=True)
        mine = optim.ShardGNMTAdam(my_model.parameters(), lr=2e-3, amsgrad=True)
    else:
        ref = torch.optim.AdamW(_groups(ref_model), lr=5e-4, foreach=False)
        mine = optim.ShardAdamW(_groups(my_model), lr=5e-4)
    for step in range(6 if kind.endswith("amsgrad") else 4):
        g = torch.Generator(device="cpu").manual_seed(step)
        # (amsgrad: the loss shrinks after the second step, so the second moment falls below its maximum)
        x = torch.randn(16, 37, generator=g).to(gpu)
        scale = 0.01 if kind.endswith("amsgrad") and step >= 2 else 1.0
        for model in (ref_model, my_model):
            model.zero_grad(set_to_none=True)
            (model(x).square().mean() * scale).backward()
        ref.step()
        mine.step()
        torch.cuda.synchronize()
        for pr, pm in zip(ref_model.parameters(), my_model.parameters()):
            assert _close(pm, pr, 1e-6, 1e-8), f"{kind} step {step}"
    key = "momentum_buffer" if kind.startswith("sgd") else "exp_avg"
    for pr, pm in zip(ref_model.parameters(), my_model.parameters()):
        assert _close(mine.state[pm][key], ref.state[pr][key], 1e-6, 1e-8)
        if kind.endswith("amsgrad"):
            assert _close(mine.state[pm]["max_exp_avg_sq"], ref.state[pr]["max_exp_avg_sq"], 1e-6, 1e-14)
            assert bool((mine.state[pm]["max_exp_avg_sq"] >= mine.state[pm]["exp_avg_sq"]).all())
    if kind.endswith("amsgrad"):
        above = torch.cat([(mine.state[p]["max_exp_avg_sq"] > mine.state[p]["exp_avg_sq"]).reshape(-1) for p in my_model.parameters()])
        assert bool(above.any())                             # somewhere the maximum did part from the moment


def test_shard_step_with_bucket_gradients_updates_only_matching_parameters(gpu):
    from jabas_amd import optim
    from jabas_amd.train.trainer import tag_parameter_indices
    model = tag_parameter_indices(_mlp(1).to(gpu))
    ref_model = copy.deepcopy(model)
    params = list(model.parameters())
    opt = optim.ShardAdamW(_groups(model), lr=5e-4)
    ref = torch.optim.AdamW(_groups(ref_model), lr=5e-4, foreach=False)
    before = [p.detach().clone() for p in params]
    # a "bucket": one flat buffer carrying the gradients of parameters 2..5, views tagged by index;
    # parameter 3 has 33 elements, so the views after it start off a 16-byte line
    chosen = [2, 3, 4, 5]
    flat = torch.randn(sum(params[i].numel() for i in chosen), device=gpu) * 1e-2
    grads, off = [], 0
    for i in chosen:
        v = flat[off:off + params[i].numel()].view_as(params[i])
        v.index = i
        grads.append(v)
        off += params[i].numel()
    opt.step(grads)
    torch.cuda.synchronize()
    for i, (p, rp) in enumerate(zip(params, ref_model.parameters())):
        rp.grad = grads[chosen.index(i)].clone() if i in chosen else None
    ref.step()
    for i, (p, rp) in enumerate(zip(params, ref_model.parameters())):
        if i in chosen:
            assert _close(p, rp, 1e-6, 1e-8), i
            assert not torch.equal(p, before[i])
        else:
            assert torch.equal(p, before[i]), i
            assert len(opt.state[p]) == 0


@pytest.mark.parametrize("kind", ["sgd", "adamw", "gnmt_adam"])
def test_shard_optimizers_refresh_the_other_replicas_in_the_same_launch(gpu, kind):
    """``attach_replicas``: the weights of the other VSWs' models follow the main model's bit for bit after
    every ``step()`` and ``step(bucket gradients)``, through first and remembered calls, for a replica whose
    tensors sit at another position of a 16-byte line too (copied after the launch); the main model itself
    steps exactly as it does without replicas; detaching stops the refresh."""
    from jabas_amd import optim
    from jabas_amd.train.trainer import tag_parameter_indices
    main, alone = tag_parameter_indices(_mlp(3).to(gpu)), tag_parameter_indices(_mlp(3).to(gpu))
    rep1, rep2 = _mlp(3).to(gpu), _mlp(3).to(gpu)
    # replica 2's parameters are views that start one element into their own buffers: not congruent with the main ones
    for q in rep2.parameters():
        buf = torch.zeros(q.numel() + 1, device=gpu)
        view = buf[1:].view(q.shape)
        view.copy_(q.data)
        q.data = view

    def build(model):
        if kind == "sgd":
            return optim.ShardSGD(_groups(model), lr=0.1, momentum=0.9)
        if kind == "adamw":
            return optim.ShardAdamW(_groups(model), lr=5e-4)
        return optim.ShardGNMTAdam(list(model.parameters()), lr=2e-3, grad_clip=0.05)
    mine, ref = build(main), build(alone)
    assert mine.attach_replicas(main.parameters(), rep1.parameters(), rep2.parameters()) is mine
    params = list(main.parameters())
    for step in range(6):
        gen = torch.Generator().manual_seed(40 + step)
        grads = [(torch.randn(p.shape, generator=gen) * 1e-2).to(gpu) for p in params]
        if step % 2 == 0:                                    # every parameter from its .grad
            for m in (main, alone):
                for p, g in zip(m.parameters(), grads):
                    p.grad = g.clone()
            mine.step()
            ref.step()
            touched = range(len(params))
        else:                                                # one "bucket": parameters 1..3
            touched = [1, 2, 3]
            for opt_, m in ((mine, main), (ref, alone)):
                views = []
                for i in touched:
                    v = grads[i].clone()
                    v.index = i
                    views.append(v)
                opt_.step(views)
        torch.cuda.synchronize()
        for i, (p, a, q1, q2) in enumerate(zip(params, alone.parameters(), rep1.parameters(), rep2.parameters())):
            assert torch.equal(p, a), (kind, step, i)                            # replicas change nothing for the main model
            if i in touched or step > 0:
                assert torch.equal(q1, p) and torch.equal(q2, p), (kind, step, i)
    mine.attach_replicas()
    before = [q.detach().clone() for q in rep1.parameters()]
    for p in main.parameters():
        p.grad = torch.ones_like(p) * 1e-2
    mine.step()
    torch.cuda.synchronize()
    assert all(torch.equal(q, b) for q, b in zip(rep1.parameters(), before))
    assert not torch.equal(params[0], before[0])
    with pytest.raises(ValueError):
        mine.attach_replicas(main.parameters(), list(rep1.parameters())[:-1])
    with pytest.raises(ValueError):
        mine.attach_replicas(main.parameters(), main.parameters())
    with pytest.raises(ValueError):
        mine.attach_replicas(list(main.parameters())[1:], list(rep1.parameters())[1:])


@pytest.mark.parametrize("level,batches,gdt", [("full", (4, 2, 2), torch.float32), ("gram", (4, 2, 2), torch.float32),
                                               ("gram", (64, 56, 48, 40, 32, 24, 16, 8), torch.bfloat16)])
@pytest.mark.parametrize("deferred", [False, True])
def test_k_vsw_rendezvous_with_streams_and_threads(gpu, deferred, level, batches, gdt):
    """K hook threads on K streams hand their buckets over in different orders. Per-bucket mode: the
    last arrival queues that bucket's launch. Deferred mode: nothing is queued until finish_step, which
    queues one planned launch over all buckets (built once, reused while DDP hands over the same buffers).
    Level 'gram': the rows also carry the products of every pair of VSWs' gradients (the Gram matrix over
    all buckets against the float64 oracle's), for three fp32 VSWs and for eight with bf16 buckets (statistics
    only there: without an optimizer bound nothing holds a reduced-precision bucket's fp32 aggregate)."""
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync

    class Bucket:
        def __init__(self, i, t):
            self._i, self._t = i, t

        def index(self):
            return self._i

        def buffer(self):
            return self._t

    K, sizes = len(batches), [40001, 7, 250000]
    tol = 1e-6 if gdt == torch.float32 else 1e-5
    local = LocalBucketSync(batches, deferred=deferred, stats_level=level)
    st = H.GradientSimilarityState(None, K + K % 2, None, [], 1).attach_local(local)
    main_hook = H.similimarity_allreduce_hook(H.subgroup_allreduce_hook)
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    dev = [[torch.empty(n, dtype=gdt, device=gpu) for _ in range(K)] for n in sizes]      # DDP's bucket buffers: the same every step
    plans = []
    for step in range(3):
        host = [[(torch.randn(n, generator=torch.Generator().manual_seed(1000 * step + 100 * b + k)) * 1e-3).to(gdt)
                 for k in range(K)] for b, n in enumerate(sizes)]
        futs = {}

        def vsw(k):
            with torch.cuda.stream(streams[k]):
                order = range(len(sizes)) if k % 2 == 0 else reversed(range(len(sizes)))
                for b in order:
                    dev[b][k].copy_(host[b][k])                               # "backward" fills the bucket on this stream
                    bucket = Bucket(b, dev[b][k])
                    futs[(k, b)] = main_hook(st, bucket) if k == 0 else H.dummy_hook(H.VSWPeerState(local, k), bucket)

        threads = [threading.Thread(target=vsw, args=(k,)) for k in range(K)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        for f in futs.values():
            f.wait()
        before = local.launched
        local.finish_step(streams)
        assert local.launched - before == (1 if deferred else 0)
        assert local.launched == (step + 1) * (1 if deferred else len(sizes))
        plans.append(local._plan)
        torch.cuda.synchronize()
        for b in range(len(sizes)):
            if gdt == torch.float32:
                want = O.aggregate(host[b], batches)
                assert torch.equal(dev[b][0].cpu().view(torch.int32), want.view(torch.int32)), (step, b)
            for k in range(0 if gdt != torch.float32 else 1, K):
                assert torch.equal(dev[b][k].cpu().float(), host[b][k].float())
        rows = {s.index: s.cpu() for s in st.grad_placeholder}
        assert sorted(rows) == [0, 1, 2]
        for b in range(len(sizes)):
            want = O.stats(host[b], batches)
            assert _close(rows[b][1:4 + K], want[1:4 + K], tol, 0.0)
            assert abs(float(rows[b][0] - want[0])) <= tol * float(torch.sqrt(want[1] * want[2]))
        whole = O.cosine_from_rows(torch.stack([O.stats(host[b], batches) for b in range(len(sizes))]))
        assert H.cosine_similarity_from_placeholder(st.grad_placeholder) == pytest.approx(whole, rel=1e-9 if gdt == torch.float32 else 1e-4, abs=1e-5)
        width = 4 + K + (K * (K - 1) // 2 if level == "gram" else 0)
        assert all(torch.count_nonzero(r[width:]) == 0 for r in rows.values())
        if level == "gram":
            from jabas_amd import sync
            got = sync.gram_from_stats(torch.stack([rows[b] for b in range(len(sizes))]), K)
            want = O.gram([torch.cat([host[b][k] for b in range(len(sizes))]) for k in range(K)])
            scale = torch.sqrt(torch.outer(torch.diagonal(want), torch.diagonal(want)))
            assert bool(((got - want).abs() <= (1e-11 if gdt == torch.float32 else 1e-5) * scale).all())
        st.grad_placeholder.clear()
        st.step += 1
    if deferred:
        assert plans[0] is not None and plans[1] is plans[0] and plans[2] is plans[0]


@pytest.mark.parametrize("share,keep_grads", [(True, False), (False, False), (True, True)])
@pytest.mark.parametrize("kind", ["sgd", "adamw"])
def test_trainer_end_to_end_matches_plain_torch_step(gpu, kind, share, keep_grads):
    """keep_grads: after a step the main model's .grad holds the synchronised gradient, as the reference leaves it
    in the main VSW; by default .grad is None after a step (the launch writes the aggregate nowhere)."""
    from jabas_amd.train import VSWSyncTrainer
    batches = (6, 2)
    if kind == "sgd":
        opt = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                   groups=[dict(lr=0.05, weight_decay=0.0), dict(lr=0.05, weight_decay=0.05)])
    else:
        opt = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
                   groups=[dict(lr=1e-3, weight_decay=0.0), dict(lr=1e-3, weight_decay=0.05)])
    crit = torch.nn.MSELoss()
    trainer = VSWSyncTrainer(gpu, batches, opt, interval=2, param_groups_func=_groups, share_weights=share,
                             keep_grads=keep_grads)
    trainer.prepare_stream_parallel(_mlp(3), crit)
    # one weight arena for every VSW's model, or one per VSW refreshed by the launch
    assert len(trainer.engine.fanout) == (0 if share else 1)
    for p, q in zip(trainer.main_model.parameters(), trainer.local_models[1].parameters()):
        assert (p.data_ptr() == q.data_ptr()) == share and p is not q
    ref_model = _mlp(3).to(gpu)
    groups = _groups(ref_model)
    if kind == "sgd":
        ref_opt = torch.optim.SGD(groups, lr=0.05, momentum=0.9, foreach=False)
    else:
        ref_opt = torch.optim.AdamW(groups, lr=1e-3, foreach=False)
    w, _, _ = O.batch_weights(batches)
    for step in range(1, 5):
        gen = torch.Generator().manual_seed(step)
        data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu)) for b in batches]
        trainer.compute(data)
        # plain torch: per-VSW gradients with the same weights, batch-weighted sum, optimizer step
        per_vsw = []
        for x, y in data:
            ref_model.zero_grad(set_to_none=True)
            crit(ref_model(x), y).backward()
            per_vsw.append([p.grad.detach().clone() for p in ref_model.parameters()])
        for i, p in enumerate(ref_model.parameters()):
            p.grad = torch.add(torch.mul(per_vsw[0][i], w[0]), torch.mul(per_vsw[1][i], w[1]))
        if trainer.similarity_state.step % 2 == 0:
            flat = [torch.cat([g.reshape(-1) for g in gs]) for gs in per_vsw]
            want_cos = torch.nn.functional.cosine_similarity(flat[0].double(), flat[1].double(), dim=0).item()
        ref_opt.step()
        stat_step = trainer.similarity_state.step % 2 == 0
        trainer.step()
        torch.cuda.synchronize()
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 1e-6, 1e-7), f"{kind} step {step}"
            if keep_grads:
                assert _close(p.grad, rp.grad, 1e-5, 1e-7), f"{kind} step {step}: synchronised gradient"
            else:
                assert p.grad is None
        for m in trainer.local_models[1:]:
            for p, q in zip(m.parameters(), trainer.main_model.parameters()):
                assert torch.equal(p, q)                       # replicas refreshed by the same launch
        if stat_step:
            assert float(trainer.cos_placeholder) == pytest.approx(want_cos, rel=1e-6)
    assert trainer.similarity_state.step == 5


def test_trainer_adds_and_removes_workers_from_the_similarity(gpu):
    from jabas_amd.train import VSWSyncTrainer
    from jabas_amd.train.adaptive import AdaptiveBatchController
    import math
    opt = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
               groups=[dict(lr=0.05, weight_decay=0.0), dict(lr=0.05, weight_decay=0.05)])
    crit = torch.nn.MSELoss()
    ctl = AdaptiveBatchController(8, 4, similarity_target=2.0, adjust_rate=0.1)     # cos < 2 always: grow
    trainer = VSWSyncTrainer(gpu, (4, 4), opt, interval=2, param_groups_func=_groups, controller=ctl)
    trainer.prepare_stream_parallel(_mlp(5), crit)
    sizes = []
    for step in range(1, 7):
        gen = torch.Generator().manual_seed(step)
        data = [(torch.randn(4, 37, generator=gen).to(gpu), torch.randn(4, 10, generator=gen).to(gpu))
                for _ in range(trainer.num_models)]
        losses = trainer.compute(data)
        assert len(losses) == trainer.num_models
        trainer.step()
        torch.cuda.synchronize()
        sizes.append(trainer.num_models)
        for m in trainer.local_models[1:]:
            for p, q in zip(m.parameters(), trainer.main_model.parameters()):
                assert torch.equal(p, q)
    assert sizes == [2, 3, 3, 4, 4, 5]                       # statistic steps 2, 4, 6 each add a worker
    assert trainer.global_lr_modifier == pytest.approx(math.sqrt(20 / 8))
    assert trainer.similarity_state.total_num_decoupled_workers == 6      # kept even, as the reference asserts
    ctl.similarity_target = -2.0                             # cos > target always: shrink
    for step in range(7, 9):
        data = [(torch.randn(4, 37).to(gpu), torch.randn(4, 10).to(gpu)) for _ in range(trainer.num_models)]
        trainer.compute(data)
        trainer.step()
    assert trainer.num_models == 4 and len(trainer.model_streams) == 4 and trainer.engine.K == 4


@pytest.mark.parametrize("kind", ["sgd", "adamw"])
def test_trainer_steps_at_lr_times_the_controllers_modifier(gpu, kind):
    """jabas/train/trainer.py:693-700: once adaptive batching has moved the global batch size, every step
    runs at lr * global_lr_modifier (lr *= modifier before the update, /= after). Weights against a
    plain-torch optimizer driven exactly that way, while the number of VSWs changes underneath."""
    from jabas_amd.train import VSWSyncTrainer
    from jabas_amd.train.adaptive import AdaptiveBatchController
    import math
    crit = torch.nn.MSELoss()
    ctl = AdaptiveBatchController(8, 4, similarity_target=2.0, adjust_rate=0.1)     # cos < 2 always: grow
    trainer = VSWSyncTrainer(gpu, (4, 4), interval=2, controller=ctl)
    trainer.prepare_stream_parallel(_mlp(21), crit)
    ref_model = _mlp(21).to(gpu)
    if kind == "sgd":
        mine = torch.optim.SGD(_groups(trainer.main_model), lr=0.05, momentum=0.9)
        ref_opt = torch.optim.SGD(_groups(ref_model), lr=0.05, momentum=0.9, foreach=False)
    else:
        mine = torch.optim.AdamW(_groups(trainer.main_model), lr=1e-3)
        ref_opt = torch.optim.AdamW(_groups(ref_model), lr=1e-3, foreach=False)
    trainer.prepare_weight_sync_method(mine, None, _groups)
    seen = []
    for step in range(1, 7):
        K = trainer.num_models
        batches = trainer.local_batch_sizes
        modifier = trainer.global_lr_modifier
        seen.append(modifier)
        gen = torch.Generator().manual_seed(300 + step)
        data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu)) for b in batches]
        trainer.compute(data)
        w, _, _ = O.batch_weights(batches)
        per_vsw = []
        for x, y in data:
            ref_model.zero_grad(set_to_none=True)
            crit(ref_model(x), y).backward()
            per_vsw.append([p.grad.detach().clone() for p in ref_model.parameters()])
        for i, p in enumerate(ref_model.parameters()):
            acc = torch.mul(per_vsw[0][i], w[0])
            for k in range(1, K):
                acc = torch.add(acc, torch.mul(per_vsw[k][i], w[k]))
            p.grad = acc
        for g in ref_opt.param_groups:
            g["lr"] *= modifier
        ref_opt.step()
        for g in ref_opt.param_groups:
            g["lr"] /= modifier
        trainer.step()
        torch.cuda.synchronize()
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 1e-6, 1e-7), f"{kind} step {step} modifier {modifier}"
    assert seen[0] == 1.0 and seen[-1] == pytest.approx(math.sqrt(16 / 8)) and len(set(seen)) >= 3
    assert mine.param_groups[0]["lr"] == (0.05 if kind == "sgd" else 1e-3)      # the caller's lr itself is left alone


@pytest.mark.parametrize("kind", ["sgd", "adamw", "shard_adam", "adamw_amsgrad"])
def test_trainer_takes_the_callers_optimizer_and_scheduler(gpu, kind):
    """The reference's order of calls (examples/resnet50/main.py:351-366, examples/vit/main.py:425-478):
    prepare_stream_parallel, an optimizer built over trainer.main_model, prepare_weight_sync_method
    (optimizer, scheduler), then learning rates driven through trainer.main_optimizer.param_groups."""
    from jabas_amd.train import VSWSyncTrainer
    from jabas_amd import optim
    batches = (5, 3)
    crit = torch.nn.MSELoss()
    trainer = VSWSyncTrainer(gpu, batches, interval=2)
    trainer.prepare_stream_parallel(_mlp(11), crit)
    ref_model = _mlp(11).to(gpu)

    def build(model, shard):
        groups = _groups(model)
        if kind == "sgd":
            return torch.optim.SGD(groups, lr=0.05, momentum=0.9, foreach=False)
        if kind == "adamw":
            return torch.optim.AdamW(groups, lr=1e-3, foreach=False)
        if kind == "adamw_amsgrad":
            return torch.optim.AdamW(groups, lr=1e-3, foreach=False, amsgrad=True)
        return (optim.ShardAdam if shard else torch.optim.Adam)(groups, lr=2e-3, **({} if shard else {"foreach": False}))

    mine, ref_opt = build(trainer.main_model, True), build(ref_model, False)
    lam = lambda it: 1.0 / (1.0 + 0.5 * it)
    sched = torch.optim.lr_scheduler.LambdaLR(mine, lam) if kind != "sgd" else None
    ref_sched = torch.optim.lr_scheduler.LambdaLR(ref_opt, lam) if kind != "sgd" else None
    trainer.prepare_weight_sync_method(mine, sched, _groups)
    assert trainer.main_optimizer is mine and trainer.local_optimizers == [mine]
    w, _, _ = O.batch_weights(batches)
    for step in range(1, 6):
        if kind == "sgd":                                   # the reference's lr policy writes param_groups directly
            for opt_ in (trainer.main_optimizer, ref_opt):
                for g in opt_.param_groups:
                    g["lr"] = 0.05 * (0.8 ** step)
        gen = torch.Generator().manual_seed(70 + step)
        shrink = 0.01 if kind.endswith("amsgrad") and step >= 3 else 1.0    # the second moment falls below its maximum
        data = [(torch.randn(b, 37, generator=gen).to(gpu) * shrink, torch.randn(b, 10, generator=gen).to(gpu) * shrink)
                for b in batches]
        trainer.compute(data)
        per_vsw = []
        for x, y in data:
            ref_model.zero_grad(set_to_none=True)
            crit(ref_model(x), y).backward()
            per_vsw.append([p.grad.detach().clone() for p in ref_model.parameters()])
        for i, p in enumerate(ref_model.parameters()):
            p.grad = torch.add(torch.mul(per_vsw[0][i], w[0]), torch.mul(per_vsw[1][i], w[1]))
        ref_opt.step()
        if ref_sched is not None:
            ref_sched.step()
        trainer.step()
        torch.cuda.synchronize()
        assert trainer.sync_step == step
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 1e-6, 1e-7), f"{kind} step {step}"
        if ref_sched is not None:
            assert mine.param_groups[0]["lr"] == pytest.approx(ref_opt.param_groups[0]["lr"], rel=1e-12)
    # the caller's optimizer object shows the state the fused launch maintains
    sd = mine.state_dict()
    assert len(sd["state"]) == len(list(trainer.main_model.parameters()))
    key = "momentum_buffer" if kind == "sgd" else "exp_avg"
    seen = _states(mine)
    for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
        assert _close(seen[id(p)][key], ref_opt.state[rp][key], 1e-6, 1e-8)
        if kind != "sgd":
            assert float(mine.state[p]["step"]) == 5.0
            assert _close(seen[id(p)]["exp_avg_sq"], ref_opt.state[rp]["exp_avg_sq"], 1e-6, 1e-12)
            # interleaved moments (the trainer's default): copies for state_dict() only, none kept in between
            assert "exp_avg" not in mine.state[p] and not trainer.engine.state_is_live
        if kind.endswith("amsgrad"):
            assert _close(seen[id(p)]["max_exp_avg_sq"], ref_opt.state[rp]["max_exp_avg_sq"], 1e-6, 1e-12)


@pytest.mark.parametrize("kind", ["sgd", "adamw"])
def test_trainer_follows_a_scheduler_that_cycles_the_momentum(gpu, kind):
    """torch's OneCycleLR moves the momentum (SGD) or beta1 (Adam kinds) of every group along with the learning
    rate: the launch takes them from the optimizer object at every step, like the learning rate."""
    from jabas_amd.train import VSWSyncTrainer
    batches = (5, 3)
    crit = torch.nn.MSELoss()
    trainer = VSWSyncTrainer(gpu, batches, interval=100)
    trainer.prepare_stream_parallel(_mlp(12), crit)
    ref_model = _mlp(12).to(gpu)

    def build(model):
        if kind == "sgd":
            return torch.optim.SGD(_groups(model), lr=0.05, momentum=0.9, foreach=False)
        return torch.optim.AdamW(_groups(model), lr=1e-3, foreach=False)

    def cycle(o):
        return torch.optim.lr_scheduler.OneCycleLR(o, max_lr=0.08 if kind == "sgd" else 4e-3, total_steps=8,
                                                   base_momentum=0.6, max_momentum=0.95)

    mine, ref_opt = build(trainer.main_model), build(ref_model)
    sched, ref_sched = cycle(mine), cycle(ref_opt)
    trainer.prepare_weight_sync_method(mine, sched, _groups)
    w, _, _ = O.batch_weights(batches)
    seen = set()
    for step in range(1, 7):
        gen = torch.Generator().manual_seed(170 + step)
        data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu)) for b in batches]
        trainer.compute(data)
        per_vsw = []
        for x, y in data:
            ref_model.zero_grad(set_to_none=True)
            crit(ref_model(x), y).backward()
            per_vsw.append([p.grad.detach().clone() for p in ref_model.parameters()])
        for i, p in enumerate(ref_model.parameters()):
            p.grad = torch.add(torch.mul(per_vsw[0][i], w[0]), torch.mul(per_vsw[1][i], w[1]))
        seen.add(mine.param_groups[0]["momentum"] if kind == "sgd" else mine.param_groups[0]["betas"][0])
        ref_opt.step()
        ref_sched.step()
        trainer.step()
        torch.cuda.synchronize()
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 1e-6, 1e-7), f"{kind} step {step}"
    assert len(seen) >= 5                                   # the momentum did move
    # groups that come to differ in it cannot share a launch
    if kind == "sgd":
        mine.param_groups[1]["momentum"] = 0.5
    else:
        mine.param_groups[1]["betas"] = (0.5, 0.999)
    trainer.compute(data)
    with pytest.raises(ValueError, match="parameter groups differ"):
        trainer.step()


def test_trainer_rejects_optimizers_it_cannot_mirror(gpu):
    from jabas_amd.train import VSWSyncTrainer
    trainer = VSWSyncTrainer(gpu, (2, 2))
    with pytest.raises(RuntimeError):
        trainer.prepare_weight_sync_method(None)
    trainer.prepare_stream_parallel(_mlp(1), torch.nn.MSELoss())
    with pytest.raises(TypeError):
        trainer.prepare_weight_sync_method(torch.optim.RMSprop(trainer.main_model.parameters(), lr=0.1))
    with pytest.raises(ValueError):
        trainer.prepare_weight_sync_method(torch.optim.Adam(trainer.main_model.parameters(), lr=0.1, maximize=True))
    groups = _groups(trainer.main_model)
    groups[0]["momentum"] = 0.5
    with pytest.raises(ValueError):
        trainer.prepare_weight_sync_method(torch.optim.SGD(groups, lr=0.1, momentum=0.9))
    with pytest.raises(ValueError):                         # a parameter outside every group
        trainer.prepare_weight_sync_method(torch.optim.SGD(list(trainer.main_model.parameters())[:2], lr=0.1))


def test_trainer_accumulates_micro_batches_between_steps(gpu):
    """compute() twice, then step(): every VSW's bucket holds the sum of two micro-batch gradients, the
    step divides by the number of accumulated micro-batches (IIDP's accum_step + 1)."""
    from jabas_amd.train import VSWSyncTrainer
    batches = (4, 2)
    crit = torch.nn.MSELoss()
    trainer = VSWSyncTrainer(gpu, batches, interval=1)
    trainer.prepare_stream_parallel(_mlp(21), crit)
    mine = torch.optim.SGD(_groups(trainer.main_model), lr=0.05, momentum=0.9, foreach=False)
    trainer.prepare_weight_sync_method(mine, None, _groups)
    ref_model = _mlp(21).to(gpu)
    ref_opt = torch.optim.SGD(_groups(ref_model), lr=0.05, momentum=0.9, foreach=False)
    w, _, _ = O.batch_weights(batches, accumulations=2)
    for step in range(1, 4):
        sums = None
        for micro in range(2):
            gen = torch.Generator().manual_seed(1000 * step + micro)
            data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu))
                    for b in batches]
            trainer.compute(data)
            per_vsw = []
            for x, y in data:
                ref_model.zero_grad(set_to_none=True)
                crit(ref_model(x), y).backward()
                per_vsw.append([p.grad.detach().clone() for p in ref_model.parameters()])
            sums = per_vsw if sums is None else [[a + b for a, b in zip(s, g)] for s, g in zip(sums, per_vsw)]
        assert trainer.accumulated == 2
        for i, p in enumerate(ref_model.parameters()):
            p.grad = torch.add(torch.mul(sums[0][i], w[0]), torch.mul(sums[1][i], w[1]))
        ref_opt.step()
        trainer.step()
        torch.cuda.synchronize()
        assert trainer.accumulated == 0
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 1e-6, 1e-7), step


@pytest.mark.parametrize("kind,interleave", [("sgd", True), ("adamw", True), ("adamw_amsgrad", True), ("adamw", False),
                                             ("adamw_amsgrad", False)])
def test_trainer_resumes_bit_for_bit_from_its_checkpoint(gpu, kind, interleave, tmp_path):
    """state_dict() after 3 steps, through a file, into a fresh trainer (other initial weights, another
    number of VSWs): the next 3 steps give the bits of the uninterrupted run. The optimizer entry is in
    torch's own format: a stock torch optimizer loads it. With Adam's moments interleaved in one arena (the
    default) and with flat state arenas, whose views the optimizer object then holds at all times."""
    from jabas_amd.train import VSWSyncTrainer
    batches = (4, 4, 4)
    crit = torch.nn.MSELoss()

    def make(seed, n_vsw):
        t = VSWSyncTrainer(gpu, (4,) * n_vsw, interval=2, interleave_moments=interleave)
        t.prepare_stream_parallel(_mlp(seed), crit)
        if kind == "sgd":
            o = torch.optim.SGD(_groups(t.main_model), lr=0.05, momentum=0.9, foreach=False)
        else:
            o = torch.optim.AdamW(_groups(t.main_model), lr=1e-3, foreach=False, amsgrad=kind.endswith("amsgrad"))
        sch = torch.optim.lr_scheduler.LambdaLR(o, lambda it: 1.0 / (1.0 + 0.25 * it))
        t.prepare_weight_sync_method(o, sch)
        return t, o

    def run(t, first, last):
        for step in range(first, last + 1):
            gen = torch.Generator().manual_seed(900 + step)
            data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu))
                    for b in batches]
            t.compute(data)
            t.step()
        torch.cuda.synchronize()

    a, opt_a = make(21, 3)
    run(a, 1, 3)
    path = tmp_path / "trainer.pth"
    torch.save(a.state_dict(), path)
    run(a, 4, 6)

    b, opt_b = make(22, 2)                                # other weights, 2 VSWs: both replaced by the checkpoint
    b.load_state_dict(torch.load(path, map_location=gpu, weights_only=True))
    assert b.num_models == 3 and b.sync_step == 3 and b.engine.step_count == 3
    base_lr = 0.05 if kind == "sgd" else 1e-3
    assert opt_b.param_groups[0]["lr"] == pytest.approx(base_lr / (1.0 + 0.25 * 3), rel=1e-12)
    run(b, 4, 6)
    assert b.sync_step == a.sync_step == 6
    for pa, pb in zip(a.main_model.parameters(), b.main_model.parameters()):
        assert torch.equal(pa.detach().view(torch.int32), pb.detach().view(torch.int32))
    for m in b.local_models[1:]:
        for pm, pb in zip(m.parameters(), b.main_model.parameters()):
            assert torch.equal(pm, pb)
    keys = ("momentum_buffer",) if kind == "sgd" else ("exp_avg", "exp_avg_sq") + (("max_exp_avg_sq",) if kind.endswith("amsgrad") else ())
    live = b.engine.state_is_live
    assert live == (kind == "sgd" or not interleave)
    arenas = {"momentum_buffer": b.engine.state1, "exp_avg": b.engine.state1, "exp_avg_sq": b.engine.state2,
              "max_exp_avg_sq": b.engine.state3}
    seen_a, seen_b = _states(opt_a), _states(opt_b)
    for pa, pb in zip(a.main_model.parameters(), b.main_model.parameters()):
        for key in keys:
            assert torch.equal(seen_a[id(pa)][key], seen_b[id(pb)][key])
            if live:                                                                 # still views of the arenas
                assert torch.equal(opt_a.state[pa][key], opt_b.state[pb][key])
                assert opt_b.state[pb][key].untyped_storage().data_ptr() == arenas[key].untyped_storage().data_ptr()
            else:                                                                    # copies for state_dict() only
                assert key not in opt_b.state[pb]
    assert opt_a.param_groups[0]["lr"] == opt_b.param_groups[0]["lr"]

    # a stock torch optimizer over a plain copy of the model takes the optimizer entry as it is
    plain = _mlp(5).to(gpu)
    plain.load_state_dict(b.state_dict()["model"])
    stock = (torch.optim.SGD(_groups(plain), lr=0.05, momentum=0.9) if kind == "sgd"
             else torch.optim.AdamW(_groups(plain), lr=1e-3, amsgrad=kind.endswith("amsgrad")))
    stock.load_state_dict(b.state_dict()["optimizer"])
    for pp, pb in zip(plain.parameters(), b.main_model.parameters()):
        assert torch.equal(stock.state[pp][keys[0]], seen_b[id(pb)][keys[0]])

    # and the other way round: a checkpoint of a plain torch run (no trainer entries) resumes here
    c, opt_c = make(23, 3)
    c.load_state_dict({"model": plain.state_dict(), "optimizer": stock.state_dict()})
    assert c.engine.step_count == (1 if kind == "sgd" else 6)
    for pc, pb in zip(c.main_model.parameters(), b.main_model.parameters()):
        assert torch.equal(pc, pb)
        for key in keys:
            assert torch.equal(_states(opt_c)[id(pc)][key], seen_b[id(pb)][key])

    # loading into the caller's own optimizer object is enough: the loaded tensors reach the arenas (a hook on the
    # optimizer), so with the weights put back a run continues as the one that was saved did
    d, opt_d = make(21, 3)
    run(d, 1, 5)                                          # somewhere else: its state must be replaced, not kept
    saved = torch.load(path, map_location=gpu, weights_only=True)
    with torch.no_grad():
        for m in d.local_models:
            m.load_state_dict(saved["model"])
    opt_d.load_state_dict(saved["optimizer"])
    assert d.engine.step_count == (1 if kind == "sgd" else 3)
    d.sync_step, d.similarity_state.step = saved["sync_step"], saved["similarity_step"]
    for sch, sd in zip(d.local_schedulers, saved["schedulers"]):
        sch.load_state_dict(sd)
    run(d, 4, 6)
    for pa, pd in zip(a.main_model.parameters(), d.main_model.parameters()):
        assert torch.equal(pa.detach().view(torch.int32), pd.detach().view(torch.int32))
    seen_d = _states(opt_d)
    for pa, pd in zip(a.main_model.parameters(), d.main_model.parameters()):
        for key in keys:
            assert torch.equal(seen_a[id(pa)][key], seen_d[id(pd)][key])


def test_trainer_with_bf16_gradient_buckets(gpu):
    """Reduced-precision buckets (the ViT-L/16 configuration): every VSW's gradient is rounded to bf16
    into its bucket (added in bf16 on further micro-batches), the aggregate and AdamW run in fp32. The
    buckets are not cleared between steps: the first micro-batch of a step overwrites them."""
    from jabas_amd.train import VSWSyncTrainer
    batches = (6, 2)
    crit = torch.nn.MSELoss()
    trainer = VSWSyncTrainer(gpu, batches, interval=1, grad_dtype=torch.bfloat16)
    trainer.prepare_stream_parallel(_mlp(31), crit)
    mine = torch.optim.AdamW(_groups(trainer.main_model), lr=2e-3, foreach=False)
    trainer.prepare_weight_sync_method(mine)
    ref_model = _mlp(31).to(gpu)
    ref_opt = torch.optim.AdamW(_groups(ref_model), lr=2e-3, foreach=False)
    for step, micro in ((1, 1), (2, 2), (3, 1)):
        w, _, _ = O.batch_weights(batches, accumulations=micro)
        buckets = None
        for mb in range(micro):
            gen = torch.Generator().manual_seed(500 + 10 * step + mb)
            data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu))
                    for b in batches]
            trainer.compute(data)
            fresh = []
            for x, y in data:
                ref_model.zero_grad(set_to_none=True)
                crit(ref_model(x), y).backward()
                fresh.append([p.grad.detach().to(torch.bfloat16) for p in ref_model.parameters()])
            buckets = fresh if buckets is None else [[a + b for a, b in zip(old, new)] for old, new in zip(buckets, fresh)]
        for i, p in enumerate(ref_model.parameters()):
            p.grad = torch.add(torch.mul(buckets[0][i].float(), w[0]), torch.mul(buckets[1][i].float(), w[1]))
        ref_opt.step()
        trainer.step()
        torch.cuda.synchronize()
        assert trainer.cos_placeholder is not None and -1.0 <= float(trainer.cos_placeholder) <= 1.0
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 1e-6, 1e-7), f"step {step}"
        for m in trainer.local_models[1:]:
            for pm, p in zip(m.parameters(), trainer.main_model.parameters()):
                assert torch.equal(pm, p)


@pytest.mark.parametrize("kind", ["sgd", "adamw"])
def test_shard_optimizer_remembered_calls_follow_every_change(gpu, kind):
    """step() remembers a call it has prepared once (same parameters, same gradient buffers) and then
    only refreshes launch scalars. Everything that may change between two such calls must still take
    effect: gradient values, learning rate and weight decay, gradients that need a realigned copy,
    parameters stepped in different subsets (diverging Adam step counts), a changed momentum / betas,
    and load_state_dict. Checked against torch.optim on a twin model over persistent gradient buffers."""
    from jabas_amd import optim
    from jabas_amd.train.trainer import tag_parameter_indices
    model = tag_parameter_indices(_mlp(3).to(gpu))
    ref_model = copy.deepcopy(model)
    params, ref_params = list(model.parameters()), list(ref_model.parameters())
    if kind == "sgd":
        mine = optim.ShardSGD(_groups(model), lr=0.05, momentum=0.9, weight_decay=1e-4)
        ref = torch.optim.SGD(_groups(ref_model), lr=0.05, momentum=0.9, weight_decay=1e-4, foreach=False)
    else:
        mine = optim.ShardAdamW(_groups(model), lr=1e-3)
        ref = torch.optim.AdamW(_groups(ref_model), lr=1e-3, foreach=False)
    # one flat persistent "bucket" with a view per parameter (several start off a 16-byte line)
    flat = torch.zeros(sum(p.numel() for p in params), device=gpu)
    views, off = [], 0
    for i, p in enumerate(params):
        v = flat[off:off + p.numel()].view_as(p)
        v.index = i
        views.append(v)
        off += p.numel()

    def one_step(step, subset=None):
        flat.copy_(torch.randn(flat.numel(), generator=torch.Generator().manual_seed(100 + step)) * 1e-2)
        chosen = range(len(params)) if subset is None else subset
        mine.step([views[i] for i in chosen])
        for i, rp in enumerate(ref_params):
            rp.grad = views[i].detach().clone() if i in chosen else None
        ref.step()
        torch.cuda.synchronize()
        for i, (p, rp) in enumerate(zip(params, ref_params)):
            assert _close(p, rp, 1e-6, 1e-8), (kind, step, i)

    for step in range(1, 5):                              # step 1 creates state, 2 is remembered, 3.. are replays
        one_step(step)
    assert len(mine._recipes) == 1
    for opt_ in (mine, ref):                              # a scheduler at work
        for g in opt_.param_groups:
            g["lr"] *= 0.5
        opt_.param_groups[1]["weight_decay"] = 0.02
    one_step(5)
    one_step(6)
    one_step(7, subset=[0, 1, 4])                         # a bucket's worth of parameters: its own remembered call
    one_step(8, subset=[0, 1, 4])
    one_step(9)                                           # Adam: parameters 0, 1, 4 are now two steps ahead of the rest
    one_step(10)
    if kind == "sgd":
        for opt_ in (mine, ref):
            opt_.param_groups[0]["momentum"] = 0.5        # a scalar the launches are split by
    else:
        for opt_ in (mine, ref):
            opt_.param_groups[1]["betas"] = (0.8, 0.99)
    one_step(11)
    one_step(12)
    # load_state_dict replaces the state tensors: the next call must use the restored ones, not those its
    # remembered launch pointed at (which by now hold the state after step 13)
    saved, ref_saved = copy.deepcopy(mine.state_dict()), copy.deepcopy(ref.state_dict())
    weights = [p.detach().clone() for p in params]
    one_step(13)
    mine.load_state_dict(saved)
    ref.load_state_dict(ref_saved)
    with torch.no_grad():
        for p, rp, w in zip(params, ref_params, weights):
            p.copy_(w)
            rp.copy_(w)
    one_step(14)
    one_step(15)


@pytest.mark.parametrize("max_norm", [0.05, 1e3])
def test_trainer_clips_the_global_gradient_norm(gpu, max_norm):
    """GNMT's step (examples/gnmt/seq2seq/train/trainer.py:157-161): clip_grad_norm_ over the synchronised
    gradient, then the optimizer. Against torch on a twin model; the small bound clips, the large one
    does not."""
    from jabas_amd.train import VSWSyncTrainer
    batches = (6, 2)
    crit = torch.nn.MSELoss()
    trainer = VSWSyncTrainer(gpu, batches, interval=1, clip_norm=max_norm)
    trainer.prepare_stream_parallel(_mlp(41), crit)
    mine = torch.optim.Adam(_groups(trainer.main_model), lr=2e-3, foreach=False)
    trainer.prepare_weight_sync_method(mine)
    ref_model = _mlp(41).to(gpu)
    ref_opt = torch.optim.Adam(_groups(ref_model), lr=2e-3, foreach=False)
    w, _, _ = O.batch_weights(batches)
    clipped = 0
    for step in range(1, 4):
        gen = torch.Generator().manual_seed(800 + step)
        data = [(torch.randn(b, 37, generator=gen).to(gpu), torch.randn(b, 10, generator=gen).to(gpu)) for b in batches]
        trainer.compute(data)
        per_vsw = []
        for x, y in data:
            ref_model.zero_grad(set_to_none=True)
            crit(ref_model(x), y).backward()
            per_vsw.append([p.grad.detach().clone() for p in ref_model.parameters()])
        for i, p in enumerate(ref_model.parameters()):
            p.grad = torch.add(torch.mul(per_vsw[0][i], w[0]), torch.mul(per_vsw[1][i], w[1]))
        total = torch.nn.utils.clip_grad_norm_(list(ref_model.parameters()), max_norm)
        clipped += int(float(total) > max_norm)
        ref_opt.step()
        trainer.step()
        torch.cuda.synchronize()
        for p, rp in zip(trainer.main_model.parameters(), ref_model.parameters()):
            assert _close(p, rp, 2e-6, 1e-7), f"step {step}"
    assert clipped == (3 if max_norm < 1.0 else 0)


def test_trainer_parameter_that_no_micro_batch_reaches(gpu):
    """A parameter outside the graph of a step has no gradient: its bucket slot holds zeros (not what an earlier
    step left there), so with no weight decay it stays put while the others move, across steps and across
    accumulated micro-batches."""
    from jabas_amd.train import VSWSyncTrainer

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            torch.manual_seed(9)
            self.used = torch.nn.Linear(37, 10)
            self.idle = torch.nn.Linear(37, 10)
            self.use_idle = False

        def forward(self, x):
            return self.used(x) + (self.idle(x) if self.use_idle else 0.0)

    opt = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False, groups=[dict(lr=0.05, weight_decay=0.0)])
    trainer = VSWSyncTrainer(gpu, (4, 4), opt, interval=1000)
    trainer.prepare_stream_parallel(Net(), torch.nn.MSELoss())
    main = trainer.main_model

    def iteration(micro_batches):
        for _ in range(micro_batches):
            trainer.compute([(torch.randn(4, 37, device=gpu), torch.randn(4, 10, device=gpu)) for _ in range(2)])
        trainer.step()
        torch.cuda.synchronize()

    for m in trainer.local_models:
        m.use_idle = True
    iteration(1)                                               # fills the idle layer's bucket slots with real gradients
    for m in trainer.local_models:
        m.use_idle = False
    idle_before = [p.detach().clone() for p in main.idle.parameters()]
    used_before = [p.detach().clone() for p in main.used.parameters()]
    momentum = [trainer.engine._view(trainer.engine.state1, i).clone() for i, (n, _) in enumerate(main.named_parameters())
                if n.startswith("idle")]
    iteration(1)
    iteration(2)
    assert all(not torch.equal(p, b) for p, b in zip(main.used.parameters(), used_before))
    # only the momentum of its one real step still moves the idle layer: p -= lr * (0.9 buf), then lr * (0.81 buf)
    for p, b, buf in zip(main.idle.parameters(), idle_before, momentum):
        want = b.reshape(-1) - 0.05 * (0.9 * buf) - 0.05 * (0.81 * buf)
        assert torch.allclose(p.reshape(-1), want, rtol=1e-5, atol=1e-8)
