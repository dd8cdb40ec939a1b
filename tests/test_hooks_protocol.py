"""Comm-hook protocol on the CPU: gating, placeholders, future chaining and the K-VSW
rendezvous, with fake bucket objects and a recording launcher in place of the kernel
(restated from jabas/ddp_comm_hooks/similarity_allreduce.py:8-45 and
jabas/train/trainer.py:184-195,452-468,480)."""
import random
import threading

import pytest
import torch

from jabas_amd import ddp_comm_hooks as H
from jabas_amd.local_sync import LocalBucketSync, BucketStats
from jabas_amd.train import create_optimizer_hook
from jabas_amd import optim


class NewBucket:
    """torch >= 1.10 GradBucket flavour."""

    def __init__(self, index, tensor, params=()):
        self._i, self._t, self._p = index, tensor, list(params)

    def index(self):
        return self._i

    def buffer(self):
        return self._t

    def parameters(self):
        return self._p

    def gradients(self):
        out, off = [], 0
        for p in self._p:
            out.append(self._t[off:off + p.numel()].view_as(p))
            off += p.numel()
        return out


class OldBucket:
    """torch 1.8.1 _GradBucket flavour the reference was written against."""

    def __init__(self, index, tensor):
        self._i, self._t = index, tensor

    def get_index(self):
        return self._i

    def get_tensors(self):
        return [self._t]


class Recorder:
    def __init__(self):
        self.calls = []

    def __call__(self, bucket_index, tensors, want_stats):
        self.calls.append((bucket_index, [t.clone() for t in tensors], want_stats))
        tensors[0].copy_(sum(tensors))                     # stands in for the in-place aggregate
        return torch.full((12,), float(bucket_index), dtype=torch.float64) if want_stats else None


def test_similarity_state_fields_follow_the_reference():
    st = H.GradientSimilarityState("pg", 8, "sub", [], 100)
    assert st.step == 1 and st.interval == 100
    assert st.subgroup_total_num_decoupled_workers == 4
    assert st.total_num_decoupled_workers == 8 and st.sub_group == "sub" and st.process_group == "pg"
    with pytest.raises(AssertionError):
        H.GradientSimilarityState("pg", 3, "sub", [], 100)


@pytest.mark.parametrize("make", [NewBucket, OldBucket])
def test_subgroup_hook_is_pass_through_off_interval(make):
    st = H.GradientSimilarityState(None, 2, None, [], 5)
    t = torch.arange(4.0)
    b = make(0, t)
    for step in (1, 2, 3, 4):
        st.step = step
        v = H.subgroup_allreduce_hook(st, b).wait()
        v = v[0] if isinstance(v, list) else v
        assert v is t and st.grad_placeholder == []
    assert isinstance(H.subgroup_allreduce_hook(st, OldBucket(0, t)).wait(), list)
    assert isinstance(H.subgroup_allreduce_hook(st, NewBucket(0, t)).wait(), torch.Tensor)


def test_dummy_hook_without_state_passes_the_bucket_through():
    t = torch.ones(3)
    assert H.dummy_hook(None, NewBucket(0, t)).wait() is t
    assert H.dummy_hook(None, OldBucket(0, t)).wait()[0] is t


def test_allreduce_sum_fut_single_process_is_identity():
    t = torch.ones(3)
    out = H._allreduce_sum_fut(None, t).wait()
    assert isinstance(out, list) and out[0] is t


def test_iidp_hook_needs_a_local_sync_unless_there_is_one_worker():
    t = torch.ones(3)
    assert H.iidp_allreduce_hook(H.IIDPState(None, 1), NewBucket(0, t)).wait() is t
    with pytest.raises(RuntimeError):
        H.iidp_allreduce_hook(H.IIDPState(None, 4), NewBucket(0, t))


def _wire(K, interval, recorder):
    local = LocalBucketSync([4] * K, launcher=recorder)
    st = H.GradientSimilarityState(None, K if K % 2 == 0 else K + 1, None, [], interval).attach_local(local)
    main_hook = H.similimarity_allreduce_hook(H.subgroup_allreduce_hook)
    peers = [H.VSWPeerState(local, k) for k in range(1, K)]
    return local, st, main_hook, peers


def test_main_vsw_first_does_not_block_and_fires_once_when_all_arrived():
    K, rec = 3, Recorder()
    local, st, main_hook, peers = _wire(K, 2, rec)
    grads = [torch.full((5,), float(k + 1)) for k in range(K)]
    st.step = 2                                            # statistic step
    fut0 = main_hook(st, NewBucket(7, grads[0]))
    # the Future is complete at once (DDP waits on it on the shared autograd thread); the launch is not queued yet
    assert fut0.done() and rec.calls == [] and local.pending() == [7]
    f1 = H.dummy_hook(peers[0], NewBucket(7, grads[1]))
    assert f1.done() and rec.calls == [] and st.grad_placeholder == []
    f2 = H.dummy_hook(peers[1], NewBucket(7, grads[2]))
    assert f2.done() and local.pending() == []
    assert len(rec.calls) == 1 and local.launched == 1
    idx, seen, want = rec.calls[0]
    assert idx == 7 and want is True
    assert [float(t[0]) for t in seen] == [1.0, 2.0, 3.0]   # VSW order, whatever the arrival order
    assert torch.equal(fut0.value(), torch.full((5,), 6.0)) and fut0.value() is grads[0]
    assert f1.value() is grads[1]
    assert len(st.grad_placeholder) == 1 and isinstance(st.grad_placeholder[0], BucketStats)
    assert st.grad_placeholder[0].index == 7
    local.finish_step()
    assert local.step_count == 1


def test_off_interval_steps_do_not_ask_for_statistics_nor_fill_the_placeholder():
    K, rec = 2, Recorder()
    local, st, main_hook, peers = _wire(K, 100, rec)
    for step in (1, 2, 3):
        st.step = step
        g = [torch.ones(4), torch.ones(4)]
        H.dummy_hook(peers[0], OldBucket(0, g[1]))
        out = main_hook(st, OldBucket(0, g[0])).wait()
        assert isinstance(out, list) and torch.equal(out[0], torch.full((4,), 2.0))
        local.finish_step()
    assert [c[2] for c in rec.calls] == [False, False, False]
    assert st.grad_placeholder == []


def test_trainer_side_placeholder_reset_and_step_counter():
    # the trainer empties grad_placeholder after reading it and bumps state.step (trainer.py:480,194-195)
    K, rec = 2, Recorder()
    local, st, main_hook, peers = _wire(K, 3, rec)
    stat_steps = []
    for step in range(1, 10):
        st.step = step
        for b in (0, 1):
            H.dummy_hook(peers[0], NewBucket(b, torch.ones(2)))
            main_hook(st, NewBucket(b, torch.ones(2))).wait()
        local.finish_step()
        if st.step % st.interval == 0:
            assert [s.index for s in st.grad_placeholder] == [0, 1]
            stat_steps.append(step)
            st.grad_placeholder.clear()
        else:
            assert st.grad_placeholder == []
    assert stat_steps == [3, 6, 9]


def test_threads_in_random_order_over_many_buckets():
    K, nb, rec = 4, 12, Recorder()
    local, st, main_hook, peers = _wire(K, 1, rec)
    grads = [[torch.full((3,), float(10 * b + k)) for k in range(K)] for b in range(nb)]
    futures, lock = {}, threading.Lock()

    def vsw(k):
        order = list(range(nb))
        random.Random(k).shuffle(order)
        for b in order:
            if k == 0:
                f = main_hook(st, NewBucket(b, grads[b][0]))
            else:
                f = H.dummy_hook(peers[k - 1], NewBucket(b, grads[b][k]))
            with lock:
                futures[(k, b)] = f

    threads = [threading.Thread(target=vsw, args=(k,)) for k in range(K)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert all(f.done() for f in futures.values())
    assert sorted(c[0] for c in rec.calls) == list(range(nb))
    for b in range(nb):
        assert float(grads[b][0][0]) == sum(10 * b + k for k in range(K))
    assert sorted(s.index for s in st.grad_placeholder) == list(range(nb))
    local.finish_step()


def test_finish_step_reports_missing_vsws_and_double_publish_is_an_error():
    local = LocalBucketSync([1, 1], launcher=Recorder())
    local.publish(0, 3, torch.ones(2))
    with pytest.raises(RuntimeError, match="twice"):
        local.publish(0, 3, torch.ones(2))
    with pytest.raises(ValueError):
        local.publish(2, 3, torch.ones(2))
    with pytest.raises(RuntimeError, match="not published"):
        local.finish_step()
    # a failed step leaves nothing behind: the next one starts clean
    assert local.pending() == [] and local.step_count == 0
    local.publish(0, 3, torch.ones(2))
    local.publish(1, 3, torch.ones(2))
    local.finish_step()
    assert local.step_count == 1


def test_launcher_failure_is_reported_at_the_end_of_the_step():
    def boom(*a):
        raise RuntimeError("launch refused")
    local = LocalBucketSync([1, 1], launcher=boom)
    local.publish(0, 0, torch.ones(2)).wait()
    local.publish(1, 0, torch.ones(2)).wait()
    with pytest.raises(RuntimeError, match="launch refused"):
        local.finish_step()
    local.finish_step()                                    # reported once


def test_optimizer_hook_steps_the_bucket_parameters_after_the_comm_hook():
    class FakeOpt:
        def __init__(self):
            self.seen = []

        def step(self, gradients):
            self.seen.append([(g.index, g.clone()) for g in gradients])

    p0, p1 = torch.nn.Parameter(torch.zeros(2, 2)), torch.nn.Parameter(torch.zeros(3))
    p0.index, p1.index = 5, 6
    flat = torch.arange(7.0)
    opt = FakeOpt()
    hook = create_optimizer_hook(lambda state, bucket: H.dummy_hook(None, bucket), opt)
    out = hook(None, NewBucket(0, flat, [p0, p1])).wait()
    assert out is flat
    assert [i for i, _ in opt.seen[0]] == [5, 6]
    assert torch.equal(opt.seen[0][0][1], flat[:4].view(2, 2)) and torch.equal(opt.seen[0][1][1], flat[4:])


def test_shard_optimizer_constructors_validate_like_torch():
    p = [torch.nn.Parameter(torch.zeros(4))]
    with pytest.raises(ValueError):
        optim.ShardSGD(p, lr=-1.0)
    with pytest.raises(ValueError):
        optim.ShardSGD(p, lr=0.1, momentum=0.0, nesterov=True)
    with pytest.raises(ValueError):
        optim.ShardAdam(p, betas=(1.0, 0.999))
    with pytest.raises(ValueError):
        optim.ShardAdamW(p, eps=-1e-8)
    o = optim.ShardAdamW(p)
    assert o.defaults["weight_decay"] == 1e-2 and optim.ShardAdam(p).defaults["weight_decay"] == 0
    p[0].grad = torch.ones(4)
    with pytest.raises(RuntimeError, match="GPU"):
        optim.ShardSGD(p, lr=0.1).step()                       # no CPU fallback
    g = torch.ones(4)
    with pytest.raises(ValueError, match="index"):
        optim.ShardSGD(p, lr=0.1).step([g])


def test_statistics_levels_and_their_names():
    from jabas_amd import sync, _lib as L
    assert [sync.stats_level(x) for x in (None, False, 0)] == [L.STATS_NONE] * 3
    assert [sync.stats_level(x) for x in (True, 1, "full")] == [L.STATS_FULL] * 3
    assert [sync.stats_level(x) for x in (2, "similarity")] == [L.STATS_SIMILARITY] * 2
    assert [sync.stats_level(x) for x in (3, "gram")] == [L.STATS_GRAM] * 2
    with pytest.raises(ValueError):
        sync.stats_level("everything")
    assert LocalBucketSync([1] * 4, launcher=Recorder(), stats_level="gram").stats_level == L.STATS_GRAM
    assert LocalBucketSync([1] * 8, launcher=Recorder(), stats_level="gram").stats_level == L.STATS_GRAM
    with pytest.raises(ValueError, match="up to 8"):
        LocalBucketSync([1] * 9, launcher=Recorder(), stats_level="gram")
    row = torch.arange(L.STATS_STRIDE, dtype=torch.float64)
    G = sync.gram_from_stats(torch.stack([row, row]), 3)          # slots 4..6 the norms, 7, 8, 9 the pairs (0,1) (0,2) (1,2)
    assert G.tolist() == [[8.0, 14.0, 16.0], [14.0, 10.0, 18.0], [16.0, 18.0, 12.0]]
    assert LocalBucketSync([1, 1], launcher=Recorder()).stats_level == L.STATS_SIMILARITY
    assert LocalBucketSync([1, 1], launcher=Recorder(), stats_level="full").stats_level == L.STATS_FULL
    args = sync.make_step_args((3, 1), torch.float32, stats="similarity")
    assert args.stats == L.STATS_SIMILARITY and args.K == 2


def test_optimizer_hook_needs_the_rendezvous_when_there_are_several_workers():
    """With K > 1 workers the update belongs to the launch the rendezvous queues; a hook that stepped the
    optimizer on its own would read VSW 0's bucket before the other VSWs' gradients are in it."""
    opt = torch.optim.SGD([torch.nn.Parameter(torch.zeros(3))], lr=0.1)
    hook = create_optimizer_hook(H.iidp_allreduce_hook, opt)
    with pytest.raises(RuntimeError, match="LocalBucketSync"):
        hook(H.IIDPState(None, 4), NewBucket(0, torch.ones(3)))
    # with a rendezvous attached the optimizer is bound to it and the hook is the plain hook
    local = LocalBucketSync([2, 2], launcher=Recorder())
    state = H.IIDPState(None, 2).attach_local(local)
    fut = hook(state, NewBucket(0, torch.ones(3)))
    assert fut.done() and local.optimizer is opt and local.opt["kind"] == "sgd"
    with pytest.raises(RuntimeError, match="already bound"):
        local.bind_optimizer(torch.optim.SGD([torch.nn.Parameter(torch.zeros(3))], lr=0.1))


def test_shard_gnmt_adam_constructor_follows_the_reference():
    p = [torch.nn.Parameter(torch.zeros(4)), torch.nn.Parameter(torch.zeros(2))]
    o = optim.ShardGNMTAdam(p, lr=2e-3, grad_clip=5.0)
    assert o.grad_clip == 5.0 and o.defaults["weight_decay"] == 0 and len(o.param_groups) == 1
    assert optim.ShardGNMTAdam(p).grad_clip == float("inf")
    with pytest.raises(ValueError, match="param_groups"):
        optim.ShardGNMTAdam([{"params": p[:1]}, {"params": p[1:]}], grad_clip=1.0)
    with pytest.raises(ValueError):
        optim.ShardGNMTAdam(p, betas=(0.9, 1.0))


class DDPBucket(NewBucket):
    """A GradBucket that also tells whether it is the replica's last one, as torch's does."""

    def __init__(self, index, tensor, n_buckets, params=()):
        super().__init__(index, tensor, params)
        self._n = n_buckets

    def is_last(self):
        return self._i == self._n - 1


def _reference_registration(num_models, similarity_state):
    """The shape of the reference's own wiring (jabas/train/trainer.py:452-468): the main VSW gets the
    similarity state and the chained hook, every other VSW ``None`` and ``dummy_hook``."""
    main_hook = H.similimarity_allreduce_hook(H.subgroup_allreduce_hook)
    states, hooks = [], []
    for i in range(num_models):
        if i == 0:
            states.append(similarity_state)
            hooks.append(main_hook)
        else:
            states.append(None)
            hooks.append(H.dummy_hook)
    return states, hooks


@pytest.mark.parametrize("registered", [True, False])
def test_reference_registration_none_states_find_the_meeting_point_and_the_step_ends_itself(registered):
    K, nb, rec = 3, 4, Recorder()
    local = LocalBucketSync([4] * K, launcher=rec).install("cpu")
    try:
        # the state is built exactly as the reference builds it: nobody attaches anything to it
        st = H.GradientSimilarityState(None, K + 1, None, [], 2)
        states, hooks = _reference_registration(K, st)
        assert states[1:] == [None] * (K - 1)
        params = [[torch.nn.Parameter(torch.zeros(3)) for _ in range(nb)] for _ in range(K)]
        if registered:
            class Replica:
                def __init__(self, ps):
                    self._ps = ps

                def parameters(self):
                    return iter(self._ps)
            local.register_replicas([Replica(ps) for ps in params])
        steps = (1, 2, 3)
        grads = {step: [[torch.full((3,), float(100 * step + 10 * b + k)) for k in range(K)] for b in range(nb)]
                 for step in steps}
        errors = []
        go, done = threading.Barrier(K + 1), threading.Barrier(K + 1)

        def vsw(k):                                        # one thread per VSW for the whole run, as IIDP has
            for step in steps:
                go.wait()
                try:
                    for b in range(nb):
                        fut = hooks[k](states[k], DDPBucket(b, grads[step][b][k], nb, [params[k][b]]))
                        assert fut.done()
                except Exception as exc:                   # pragma: no cover - reported below
                    errors.append(exc)
                done.wait()
        threads = [threading.Thread(target=vsw, args=(k,), daemon=True) for k in range(K)]
        for t in threads:
            t.start()
        for step in steps:
            go.wait(timeout=30)
            done.wait(timeout=30)
            assert not errors, errors
            # the last bucket's last hand-over ended the step: no call from the training loop
            assert local.step_count == step and local.pending() == []
            local.finish_step()                            # a loop that still calls it changes nothing
            assert local.step_count == step
            assert len(rec.calls) == nb * step
            for idx, seen, want in rec.calls[-nb:]:
                assert want is (step % 2 == 0)
                got = sorted(float(t[0]) for t in seen)
                assert got == [float(100 * step + 10 * idx + k) for k in range(K)]
                if registered:                             # VSW order, whatever the arrival order
                    assert [float(t[0]) for t in seen] == got
            assert len(st.grad_placeholder) == (nb if step % 2 == 0 else 0)
            st.grad_placeholder.clear()
            st.step += 1
        for t in threads:
            t.join(timeout=30)
        assert st.local is local
    finally:
        local.uninstall()
    t = torch.ones(3)
    assert H.dummy_hook(None, NewBucket(0, t)).wait() is t        # nothing installed: the pass-through again


def test_replicas_with_unequal_batches_must_be_told_apart():
    local = LocalBucketSync([4, 2], launcher=Recorder()).install("cpu")
    try:
        with pytest.raises(RuntimeError, match="register_replicas"):
            H.dummy_hook(None, NewBucket(0, torch.ones(2)))
        with pytest.raises(ValueError):
            local.register_replicas([torch.nn.Linear(2, 2)])
        a, b = torch.nn.Linear(2, 2), torch.nn.Linear(2, 2)
        local.register_replicas([a, b])
        H.dummy_hook(None, NewBucket(0, torch.ones(6), list(b.parameters())))
        assert local.pending() == [0]
        with pytest.raises(RuntimeError, match="was not told about"):
            H.dummy_hook(None, NewBucket(1, torch.ones(6), list(torch.nn.Linear(2, 2).parameters())))
    finally:
        local.uninstall()


def test_more_peers_than_the_meeting_point_expects():
    local = LocalBucketSync([1, 1], launcher=Recorder()).install("cpu")
    try:
        seen = []

        alive = threading.Barrier(2)

        def peer():
            alive.wait()                                   # both threads exist at once: two identities
            try:
                H.dummy_hook(None, NewBucket(0, torch.ones(2)))
            except RuntimeError as exc:
                seen.append(str(exc))
        threads = [threading.Thread(target=peer) for _ in range(2)]    # two peer threads, one peer slot
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert len(seen) == 1 and "more peer replicas" in seen[0]
    finally:
        local.uninstall()


def test_a_failed_launch_surfaces_in_the_hand_over_that_ends_the_step():
    """With the step ended by the last bucket's last hand-over, what went wrong in one of the step's launches is
    raised there (in training: inside that VSW's backward pass), once, and the next step starts clean."""
    calls = []

    def launcher(bucket_index, tensors, want_stats):
        calls.append(bucket_index)
        if bucket_index == 0 and len(calls) == 1:
            raise RuntimeError("launch refused")
        return None
    local = LocalBucketSync([1, 1], launcher=launcher)
    grads = [torch.ones(2), torch.ones(2)]
    for b in (0, 1):
        local.publish(0, b, grads[0], bucket=DDPBucket(b, grads[0], 2))
    local.publish(1, 0, grads[1], bucket=DDPBucket(0, grads[1], 2))           # bucket 0 complete: its launch fails
    with pytest.raises(RuntimeError, match="launch refused"):
        local.publish(1, 1, grads[1], bucket=DDPBucket(1, grads[1], 2))       # the step ends here
    assert local.step_count == 0 and local.pending() == []
    local.finish_step()                                                        # nothing left to report
    for k in (0, 1):
        for b in (0, 1):
            local.publish(k, b, grads[k], bucket=DDPBucket(b, grads[k], 2))
    assert local.step_count == 1 and calls == [0, 1, 0, 1]


def test_auto_finish_can_be_switched_off():
    local = LocalBucketSync([1, 1], launcher=Recorder(), auto_finish=False)
    for k in (0, 1):
        local.publish(k, 0, torch.ones(2), bucket=DDPBucket(0, torch.ones(2), 1))
    assert local.step_count == 0 and local.launched == 1
    local.finish_step()
    assert local.step_count == 1


def test_launch_on_last_vsw_is_a_mode_without_launch_streams():
    """The option puts launches on the VSWs' own streams: it excludes ``stream=`` (checked before any stream is
    touched), and with host tensors (no streams at all) the protocol is what it is without it."""
    with pytest.raises(ValueError, match="launch_on_last_vsw"):
        LocalBucketSync([1, 1], launcher=Recorder(), stream=object(), launch_streams=1, launch_on_last_vsw=True)
    rec = Recorder()
    local = LocalBucketSync([1, 1], launcher=rec, launch_on_last_vsw=True)
    g = [torch.full((3,), 1.0), torch.full((3,), 2.0)]
    local.publish(1, 0, g[1])
    assert rec.calls == []
    local.publish(0, 0, g[0])
    assert [c[0] for c in rec.calls] == [0] and float(g[0][0]) == 3.0
    local.finish_step()
    assert local.step_count == 1
