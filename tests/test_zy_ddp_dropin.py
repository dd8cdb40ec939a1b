"""Drop-in check with stock torch DDP on one GPU: K model replicas, each wrapped in
DistributedDataParallel (gradient_as_bucket_view=True, one process group of size 1),
driven by K threads on K streams as IIDP drives its VSWs. VSW 0 registers the similarity
hook, the others dummy_hook with a VSWPeerState (jabas/train/trainer.py:452-468); the real
GradBucket objects DDP hands to the hooks go through the fused launch. Checked against a
plain-torch batch-weighted aggregate of the same per-replica gradients.
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
    return torch.nn.Sequential(torch.nn.Linear(64, 256), torch.nn.ReLU(), torch.nn.Linear(256, 256), torch.nn.ReLU(),
                               torch.nn.Linear(256, 16))


def test_stock_ddp_buckets_through_the_hooks(gpu):
    from jabas_amd import ddp_comm_hooks as H
    from jabas_amd.local_sync import LocalBucketSync
    from torch.nn.parallel import DistributedDataParallel as DDP

    if not dist.is_initialized():
        os.environ.setdefault("MASTER_ADDR", "127.0.0.1")
        os.environ.setdefault("MASTER_PORT", "29517")
        dist.init_process_group("nccl", rank=0, world_size=1)
    K, batches = 2, (6, 2)
    crit = torch.nn.MSELoss()
    streams = [torch.cuda.Stream(gpu) for _ in range(K)]
    replicas = []
    for k in range(K):
        with torch.cuda.stream(streams[k]):
            replicas.append(DDP(_model(0).to(gpu), device_ids=[gpu.index], gradient_as_bucket_view=True,
                                bucket_cap_mb=0.1))
    torch.cuda.synchronize()
    local = LocalBucketSync(batches)
    state = H.GradientSimilarityState(dist.group.WORLD, 2, None, [], 1).attach_local(local)
    replicas[0].register_comm_hook(state=state, hook=H.similimarity_allreduce_hook(H.subgroup_allreduce_hook))
    replicas[1].register_comm_hook(state=H.VSWPeerState(local, 1), hook=H.dummy_hook)

    plain = _model(0).to(gpu)
    w, _, _ = O.batch_weights(batches)
    for step in range(1, 4):                              # step 1 is the one in which DDP rebuilds its buckets
        gen = torch.Generator().manual_seed(step)
        data = [(torch.randn(b, 64, generator=gen).to(gpu), torch.randn(b, 16, generator=gen).to(gpu)) for b in batches]
        per_vsw = []
        for x, y in data:
            plain.zero_grad(set_to_none=True)
            crit(plain(x), y).backward()
            per_vsw.append([p.grad.detach().clone() for p in plain.parameters()])
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
        local.finish_step(streams)
        torch.cuda.synchronize()
        for i, p in enumerate(replicas[0].module.parameters()):
            want = torch.add(torch.mul(per_vsw[0][i], w[0]), torch.mul(per_vsw[1][i], w[1]))
            assert torch.allclose(p.grad, want, rtol=1e-5, atol=1e-8), (step, i)
        # statistic step every step here: cosine between the two workers' whole gradients
        flat = [torch.cat([g.reshape(-1) for g in gs]).double() for gs in per_vsw]
        want_cos = torch.nn.functional.cosine_similarity(flat[0], flat[1], dim=0).item()
        got = H.cosine_similarity_from_placeholder(state.grad_placeholder)
        assert got == pytest.approx(want_cos, rel=1e-4, abs=1e-6)
        if step >= 2:                                     # DDP has rebuilt its buckets by now
            assert len(state.grad_placeholder) >= 2       # several buckets at this cap
        state.grad_placeholder.clear()
        state.step += 1
    del replicas
    dist.destroy_process_group()
