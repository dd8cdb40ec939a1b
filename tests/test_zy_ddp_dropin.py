"""Drop-in check with stock torch DDP on one GPU: K model replicas, each wrapped in
DistributedDataParallel (gradient_as_bucket_view=True, one process group of size 1),
driven by K threads on K streams as IIDP drives its VSWs. VSW 0 registers the similarity
hook, the others dummy_hook with a VSWPeerState (jabas/train/trainer.py:452-468); the real
GradBucket objects DDP hands to the hooks go through the fused launch. Checked bit for bit
against the CPU oracle fed with the very gradient bits every replica's backward left in its
bucket (VSW 0's bucket is copied by a recording hook before the launch overwrites it).
Collected late: it initialises a process group."""
import os
import threading

import pytest
import torch
import torch.distributed as dist

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _model(seed):
    torch.manual_seed(seed)
    return torch.nn.Sequential(torch.nn.Linear(64, 256), torch.nn.ReLU(), torch.nn.Linear(256, 255), torch.nn.ReLU(),
                               torch.nn.Linear(255, 16))


def _bits(t):
    return t.detach().cpu().contiguous().reshape(-1).view(torch.int32)


def _init_pg():
    if not dist.is_initialized():
        os.environ.setdefault("MASTER_ADDR", "127.0.0.1")
        os.environ.setdefault("MASTER_PORT", "29517")
        dist.init_process_group("nccl", rank=0, world_size=1)


def _replicas(gpu, K, streams):
    from torch.nn.parallel import DistributedDataParallel as DDP
    out = []
    for k in range(K):
        with torch.cuda.stream(streams[k]):
            out.append(DDP(_model(0).to(gpu), device_ids=[gpu.index], gradient_as_bucket_view=True, bucket_cap_mb=0.1))
    torch.cuda.synchronize()
    return out


class Recorder:
    """Wraps VSW 0's hook: keeps a copy of every bucket as backward left it, and which parameters it
    carries where (the launch aggregates in place into that bucket). ``hook`` is what DDP registers."""

    def __init__(self, inner, model):
        self.index_of = {id(p): i for i, p in enumerate(model.parameters())}
        self.seen = {}

        def recording_hook(state, bucket):
            buf = bucket.buffer()
            offs = [(g.data_ptr() - buf.data_ptr()) // 4 for g in bucket.gradients()]
            self.seen[bucket.index()] = (buf.clone(), [self.index_of[id(p)] for p in bucket.parameters()], offs)
            return inner(state, bucket)

        self.hook = recording_hook


def _backward_all(replicas, streams, data, crit):
    K = len(replicas)
    errors, losses = [], []
    # forward passes one after the other (DDP's forward may use the process group: bucket
    # rebuild after the first step); backward passes concurrently, one thread per VSW
    for k in range(K):
        with torch.cuda.stream(streams[k]):
            replicas[k].zero_grad(set_to_none=False)
            losses.append(crit(replicas[k](data[k][0]), data[k][1]))

    def run(k):
        try:
            with torch.cuda.stream(streams[k]):
                losses[k].backward()
        except Exception as exc:                      # pragma: no cover - reported below
            errors.append(exc)

    threads = [threading.Thread(target=run, args=(k,), daemon=True) for k in range(K)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=60)
    assert not errors, errors
    assert not any(t.is_alive() for t in threads), "a VSW thread is stuck in backward"


def _per_parameter_grads(rec, replicas):
    """[k][i]: gradient of parameter i as VSW k's backward produced it (host)."""
    n = len(rec.index_of)
    out = [[None] * n for _ in replicas]
    for (buf, idxs, offs) in rec.seen.values():
        for i, o in zip(idxs, offs):
            out[0][i] = buf[o:o + list(replicas[0].module.parameters())[i].numel()].cpu()
    for k in range(1, len(replicas)):
        for i, p in enumerate(replicas[k].module.parameters()):
            out[k][i] = p.grad.detach().reshape(-1).cpu()
    return out


@pytest.mark.parametrize("batches", [(6, 2), (6, 2, 4, 4)])
def test_stock_ddp_buckets_through_the_hooks(gpu, batches):
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync

    _init_pg()
    K = len(batches)
    crit = torch.nn.MSELoss()
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    replicas = _replicas(gpu, K, streams)
    local = LocalBucketSync(batches)
    state = H.GradientSimilarityState(dist.group.WORLD, K, None, [], 1).attach_local(local)
    rec = Recorder(H.similimarity_allreduce_hook(H.subgroup_allreduce_hook), replicas[0].module)
    replicas[0].register_comm_hook(state=state, hook=rec.hook)
    for k in range(1, K):
        replicas[k].register_comm_hook(state=H.VSWPeerState(local, k), hook=H.dummy_hook)

    for step in range(1, 4):                              # step 1 is the one in which DDP rebuilds its buckets
        gen = torch.Generator().manual_seed(step)
        data = [(torch.randn(b, 64, generator=gen).to(gpu), torch.randn(b, 16, generator=gen).to(gpu)) for b in batches]
        rec.seen.clear()
        _backward_all(replicas, streams, data, crit)
        local.finish_step()                               # the VSW streams are the ones the hooks ran on
        torch.cuda.synchronize()
        per_vsw = _per_parameter_grads(rec, replicas)
        for i, p in enumerate(replicas[0].module.parameters()):
            want = O.aggregate([per_vsw[k][i] for k in range(K)], batches)
            assert torch.equal(_bits(p.grad), _bits(want)), (step, i)
        # statistic step every step here: cosine between the batch-weighted gradients of the even and the odd workers
        halves = []
        for h in (0, 1):
            ks = [k for k in range(K) if k % 2 == h]
            tot = float(sum(batches[k] for k in ks))
            halves.append(sum(torch.cat(per_vsw[k]).double() * (batches[k] / tot) for k in ks))
        want_cos = torch.nn.functional.cosine_similarity(halves[0], halves[1], dim=0).item()
        got = H.cosine_similarity_from_placeholder(state.grad_placeholder)
        assert got == pytest.approx(want_cos, rel=1e-6 if K > 2 else 1e-9, abs=1e-9)
        if step >= 2:                                     # DDP has rebuilt its buckets by now
            assert len(state.grad_placeholder) >= 2       # several buckets at this cap
        state.grad_placeholder.clear()
        state.step += 1
    del replicas
    dist.destroy_process_group()


@pytest.mark.parametrize("kind,mode", [("sgd", "per_bucket"), ("sgd", "batched"), ("sgd", "deferred"), ("sgd", "per_bucket_shared_weights"),
                                       ("adamw", "per_bucket"), ("adamw", "batched"), ("adamw", "deferred"),
                                       ("adamw", "per_bucket_shared_weights"), ("adamw", "per_bucket_interleaved_moments"),
                                       ("adamw", "deferred_interleaved_moments")])
def test_stock_ddp_with_the_optimizer_in_the_hook(gpu, kind, mode):
    """Overlap weight-sync mode end to end with stock DDP (jabas/train/trainer.py:327-333): the optimizer
    hook on VSW 0, a launch stream of its own, the weights of both replicas and the optimizer state
    bit-exact against the oracle over four steps, across DDP's bucket rebuild after the first; one launch
    per bucket, per batch of buckets, and per step."""
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    from jabas_amd.train import prepare_overlap_optimizer_with_ddp

    _init_pg()
    K, batches = 2, (6, 2)
    crit = torch.nn.MSELoss()
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    replicas = _replicas(gpu, K, streams)
    main = replicas[0].module
    groups = [{"params": [p for p in main.parameters() if p.dim() <= 1], "weight_decay": 0.0},
              {"params": [p for p in main.parameters() if p.dim() > 1], "weight_decay": 0.05}]
    if kind == "sgd":
        optimizer = torch.optim.SGD(groups, lr=0.05, momentum=0.9)
        opt = dict(kind="sgd", momentum=0.9, dampening=0.0, nesterov=False,
                   groups=[dict(lr=0.05, weight_decay=0.0), dict(lr=0.05, weight_decay=0.05)])
    else:
        optimizer = torch.optim.AdamW(groups, lr=1e-3)
        opt = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
                   groups=[dict(lr=1e-3, weight_decay=0.0), dict(lr=1e-3, weight_decay=0.05)])
    group_of = [0 if p.dim() <= 1 else 1 for p in main.parameters()]
    p_h = [p.detach().cpu().clone().reshape(-1) for p in main.parameters()]
    s1_h, s2_h = [torch.zeros_like(p) for p in p_h], [torch.zeros_like(p) for p in p_h]

    share = mode.endswith("shared_weights")              # the replica's parameters become views of the main weight arena
    interleave = mode.endswith("interleaved_moments")    # Adam's moments of a bucket in one arena of alternating blocks
    mode = mode.replace("_interleaved_moments", "")
    local = LocalBucketSync(batches, deferred=(mode == "deferred"), batch_bytes=250_000 if mode == "batched" else 0,
                            share_weights=share, interleave_moments=interleave)
    state = H.GradientSimilarityState(dist.group.WORLD, 2, None, [], 2).attach_local(local)
    rec = Recorder(H.similimarity_allreduce_hook(H.subgroup_allreduce_hook), main)
    prepare_overlap_optimizer_with_ddp(replicas, [state, H.VSWPeerState(local, 1)], [rec.hook, H.dummy_hook], optimizer, local)
    assert local._sync_stream is not None and local.optimizer is optimizer

    for step in range(1, 5):
        for g in optimizer.param_groups:                  # a learning-rate policy writing param_groups, as the reference's do
            g["lr"] = opt["groups"][0]["lr"] * (0.9 ** (step - 1))
        gen = torch.Generator().manual_seed(40 + step)
        data = [(torch.randn(b, 64, generator=gen).to(gpu), torch.randn(b, 16, generator=gen).to(gpu)) for b in batches]
        rec.seen.clear()
        _backward_all(replicas, streams, data, crit)
        local.finish_step()
        torch.cuda.synchronize()
        per_vsw = _per_parameter_grads(rec, replicas)
        step_opt = dict(opt, groups=[dict(g, lr=g["lr"] * (0.9 ** (step - 1))) for g in opt["groups"]])
        if interleave:                                    # the moments as a checkpoint of this moment holds them
            sd_now = optimizer.state_dict()
            index = dict(zip((id(q_) for g in optimizer.param_groups for q_ in g["params"]),
                             (j for g in sd_now["param_groups"] for j in g["params"])))
        for i, (p, q) in enumerate(zip(main.parameters(), replicas[1].module.parameters())):
            agg = O.aggregate([per_vsw[0][i], per_vsw[1][i]], batches)
            O.opt_step(step_opt, group_of[i], p_h[i], agg, s1_h[i], s2_h[i], step, step == 1)
            assert torch.equal(_bits(p.grad), _bits(agg)), (step, i, "aggregate")
            assert torch.equal(_bits(p.data), _bits(p_h[i])), (step, i, "weights")
            assert torch.equal(_bits(q.data), _bits(p_h[i])), (step, i, "replica weights")
            assert (q.data_ptr() == p.data_ptr()) == share and q is not p
            st = optimizer.state[p]
            if interleave:
                assert "exp_avg" not in st and int(st["step"]) == step
                st = sd_now["state"][index[id(p)]]
            if kind == "sgd":
                assert torch.equal(_bits(st["momentum_buffer"]), _bits(s1_h[i])), (step, i)
            else:
                assert torch.equal(_bits(st["exp_avg"]), _bits(s1_h[i])), (step, i)
                assert torch.equal(_bits(st["exp_avg_sq"]), _bits(s2_h[i])), (step, i)
                assert int(st["step"]) == step
        state.grad_placeholder.clear()
        state.step += 1
    if mode == "deferred":
        assert local.launched == 4
    sd = optimizer.state_dict()                           # the caller's optimizer object checkpoints as usual
    assert len(sd["state"]) == len(p_h)
    del replicas
    dist.destroy_process_group()


class _ReferenceWiring:
    """The hook wiring of the reference's trainer, statement for statement (jabas/train/trainer.py:327-337 and
    452-468), over the attributes it reads there. What the reference reaches in its base class (IIDP's trainer,
    not part of the JABAS repository) is the three methods at the bottom."""

    def __init__(self, local_models, main_optimizer, interval, local):
        self.local_models, self.main_optimizer, self.local = local_models, main_optimizer, local
        self.num_models = self.total_num_decoupled_workers = len(local_models)
        self.interval = interval

    def _prepare_similarity_allreduce_hooks(self):
        from jabas_amd import ddp_comm_hooks as H
        self.states, self.hooks = [], []
        self.similarity_state = H.GradientSimilarityState(
            dist.group.WORLD, self.total_num_decoupled_workers, None, [], self.interval)
        subgroup_allreduce_hook = H.subgroup_allreduce_hook
        main_hook = H.similimarity_allreduce_hook(subgroup_allreduce_hook)
        dummy_hook = H.dummy_hook
        for i in range(self.num_models):
            if i == 0:
                self.states.append(self.similarity_state)
                self.hooks.append(main_hook)
            else:
                self.states.append(None)
                self.hooks.append(dummy_hook)

    def _register_comm_hook(self):
        for _, (local_model, state, hook) in enumerate(zip(self.local_models, self.states, self.hooks)):
            local_model.register_comm_hook(state=state, hook=hook)

    def _prepare_overlap_optimizer_with_ddp(self):
        self._create_stream_for_optimizer()
        self._check_overlap_with_ddp()
        for i, (local_model, state, hook) in enumerate(zip(self.local_models, self.states, self.hooks)):
            if i == 0:
                hook = self._create_optimizer_hook(hook)
            local_model.register_comm_hook(state=state, hook=hook)

    # ---- IIDP's side
    def _create_stream_for_optimizer(self):
        from jabas_amd.train import create_stream_for_optimizer
        self.local._sync_stream = create_stream_for_optimizer(next(self.local_models[0].parameters()).device)

    def _check_overlap_with_ddp(self):
        assert all(m.gradient_as_bucket_view for m in self.local_models)

    def _create_optimizer_hook(self, hook):
        from jabas_amd.train import create_optimizer_hook
        return create_optimizer_hook(hook, self.main_optimizer)


@pytest.mark.parametrize("batches,registered,overlap", [((4, 4), False, False), ((6, 2, 4, 4), True, False),
                                                        ((3, 3, 3, 3), False, True), ((6, 2), True, True)])
def test_the_references_own_registration_block_with_none_states(gpu, batches, registered, overlap):
    """Nothing of ours is handed to the hooks: the main state is built as the reference builds it, the peers
    register ``dummy_hook`` with ``state=None``, and the training loop calls neither ``attach_local`` nor
    ``finish_step``. The meeting point is found through the device (``install``, IIDP's side of the set-up),
    the VSW index through the bucket's parameters (``register_replicas``) or the hook's stream, the step ends
    with the last bucket. Aggregate (sequential mode) or weights and optimizer state (overlap mode) bit-exact
    against the oracle over four steps, across DDP's bucket rebuild."""
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync

    _init_pg()
    K = len(batches)
    crit = torch.nn.MSELoss()
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    replicas = _replicas(gpu, K, streams)
    main = replicas[0].module
    groups = [{"params": [p for p in main.parameters() if p.dim() <= 1], "weight_decay": 0.0},
              {"params": [p for p in main.parameters() if p.dim() > 1], "weight_decay": 0.05}]
    optimizer = torch.optim.AdamW(groups, lr=1e-3)
    opt = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
               groups=[dict(lr=1e-3, weight_decay=0.0), dict(lr=1e-3, weight_decay=0.05)])
    group_of = [0 if p.dim() <= 1 else 1 for p in main.parameters()]
    p_h = [p.detach().cpu().clone().reshape(-1) for p in main.parameters()]
    s1_h, s2_h = [torch.zeros_like(p) for p in p_h], [torch.zeros_like(p) for p in p_h]

    # IIDP's side of the set-up: the GPU's meeting point exists and knows the device (and, when told, the replicas)
    local = LocalBucketSync(batches, launch_streams=2).install(gpu)
    if registered:
        local.register_replicas(replicas)
    try:
        wiring = _ReferenceWiring(replicas, optimizer, 2, local)
        wiring._prepare_similarity_allreduce_hooks()
        assert wiring.states[1:] == [None] * (K - 1) and wiring.similarity_state.local is None
        rec = Recorder(wiring.hooks[0], main)              # the test's own tap on VSW 0's bucket, for the oracle
        wiring.hooks[0] = rec.hook
        if overlap:
            wiring._prepare_overlap_optimizer_with_ddp()
        else:
            wiring._register_comm_hook()
        state = wiring.similarity_state
        for step in range(1, 5):
            gen = torch.Generator().manual_seed(70 + step)
            data = [(torch.randn(b, 64, generator=gen).to(gpu), torch.randn(b, 16, generator=gen).to(gpu)) for b in batches]
            rec.seen.clear()
            _backward_all(replicas, streams, data, crit)
            assert local.step_count == step                # ended by the last bucket's last hand-over
            torch.cuda.synchronize()
            # which replica the meeting point took for which VSW index
            if registered:
                vsw_of = list(range(K))
            else:
                by_stream = {(s.stream_id, s.device_index, s.device_type): j for j, s in enumerate(streams)}
                vsw_of = [0] + [None] * (K - 1)
                for raw, k in local._stream_vsw.items():
                    vsw_of[k] = by_stream[raw]
                assert sorted(vsw_of) == list(range(K))
            per_rep = _per_parameter_grads(rec, replicas)
            per_vsw = [per_rep[j] for j in vsw_of]
            for i, p in enumerate(main.parameters()):
                agg = O.aggregate([per_vsw[k][i] for k in range(K)], batches)
                assert torch.equal(_bits(p.grad), _bits(agg)), (step, i, "aggregate")
                if overlap:
                    O.opt_step(opt, group_of[i], p_h[i], agg, s1_h[i], s2_h[i], step, step == 1)
                    assert torch.equal(_bits(p.data), _bits(p_h[i])), (step, i, "weights")
                    for r in replicas[1:]:
                        assert torch.equal(_bits(list(r.module.parameters())[i].data), _bits(p_h[i])), (step, i, "replica")
                    assert torch.equal(_bits(optimizer.state[p]["exp_avg"]), _bits(s1_h[i])), (step, i)
                    assert torch.equal(_bits(optimizer.state[p]["exp_avg_sq"]), _bits(s2_h[i])), (step, i)
            if state.step % state.interval == 0:
                halves = []
                for h in (0, 1):
                    ks = [k for k in range(K) if k % 2 == h]
                    tot = float(sum(batches[k] for k in ks))
                    halves.append(sum(torch.cat(per_vsw[k]).double() * (batches[k] / tot) for k in ks))
                want_cos = torch.nn.functional.cosine_similarity(halves[0], halves[1], dim=0).item()
                assert H.cosine_similarity_from_placeholder(state.grad_placeholder) == pytest.approx(want_cos, rel=1e-6, abs=1e-9)
            else:
                assert state.grad_placeholder == []
            state.grad_placeholder = []                    # jabas/train/trainer.py:480
            state.step += 1
        assert state.local is local and len(local._sync_streams) == (2 if overlap else 0)
    finally:
        local.uninstall()
        del replicas
        dist.destroy_process_group()
