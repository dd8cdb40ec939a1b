"""``_allreduce_sum_fut`` with a real two-rank process group (gloo, CPU tensors, loopback): the one
place where the hook layer defers to torch.distributed. With a single rank it is the identity."""
import os
import socket

import pytest
import torch
import torch.distributed as dist
import torch.multiprocessing as mp


def _free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def _rank_main(rank, world, port, out_dir):
    os.environ["MASTER_ADDR"] = "127.0.0.1"
    os.environ["MASTER_PORT"] = str(port)
    dist.init_process_group("gloo", rank=rank, world_size=world)
    try:
        from jabas_amd.ddp_comm_hooks import _allreduce_sum_fut
        t = torch.arange(8, dtype=torch.float32) * (rank + 1)
        fut = _allreduce_sum_fut(dist.group.WORLD, t)
        value = fut.wait()
        assert isinstance(value, list) and len(value) == 1
        torch.save(value[0].clone(), os.path.join(out_dir, f"rank{rank}.pt"))
    finally:
        dist.destroy_process_group()


@pytest.mark.timeout(120)
def test_allreduce_sum_fut_two_ranks_gloo(tmp_path):
    world, port = 2, _free_port()
    mp.spawn(_rank_main, args=(world, port, str(tmp_path)), nprocs=world, join=True)
    want = torch.arange(8, dtype=torch.float32) * 3.0              # rank 0 contributes x1, rank 1 x2
    for rank in range(world):
        got = torch.load(os.path.join(str(tmp_path), f"rank{rank}.pt"), weights_only=True)
        assert torch.equal(got, want), rank


def test_allreduce_sum_fut_is_the_identity_without_a_process_group():
    from jabas_amd.ddp_comm_hooks import _allreduce_sum_fut
    t = torch.randn(5)
    value = _allreduce_sum_fut(None, t).wait()
    assert isinstance(value, list) and value[0] is t
