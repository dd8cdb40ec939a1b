"""Comm hooks of similarity-based adaptive batching, same names and protocol as
jabas/ddp_comm_hooks/similarity_allreduce.py:1-45.

Protocol kept: ``state.step`` starts at 1 (skips the step in which DDP rebuilds its
buckets); a step is a statistic step when ``state.step % state.interval == 0``; on such a
step one entry per bucket is appended to ``state.grad_placeholder`` and the trainer
empties the list after reading it (jabas/train/trainer.py:184-195,480).

What changed underneath: the reference clones the bucket, sums it over a sub-group and
divides (a second copy of every gradient plus four passes); here the half-gradient
statistics come out of the same fused kernel that aggregates the bucket, so the entry
appended is a ``BucketStats`` (4 + 16 doubles on the device), not a gradient-sized tensor.
``cosine_similarity_from_placeholder`` is the matching reader.
"""
import torch

from .default_hooks import bucket_tensor, bucket_value, bucket_index, completed
from .iidp_allreduce import iidp_allreduce_hook, IIDPState
from .. import sync


class GradientSimilarityState(IIDPState):
    def __init__(self, process_group, total_num_decoupled_workers, sub_group, grad_placeholder, interval):
        super().__init__(process_group, total_num_decoupled_workers)
        self.sub_group = sub_group
        self.grad_placeholder = grad_placeholder
        assert self.total_num_decoupled_workers % 2 == 0, \
            f"self.total_num_decoupled_workers must be power of 2, but {self.total_num_decoupled_workers}"
        self.subgroup_total_num_decoupled_workers = self.total_num_decoupled_workers / 2
        self.interval = interval
        self.step = 1  # first step skipped: DDP rebuilds its buckets in it
        self._stat_buckets = set()

    def is_stat_step(self):
        return self.step % self.interval == 0


def subgroup_allreduce_hook(state, bucket):
    """Non-statistic step: pass-through. Statistic step: asks the fused launch of this
    bucket (queued by the chained all-group hook) for the half-gradient statistics."""
    tensor = bucket_tensor(bucket)
    if state.step % state.interval != 0:
        return completed(bucket_value(bucket, tensor))
    state._stat_buckets.add(bucket_index(bucket))
    return completed(bucket_value(bucket, tensor))


def similimarity_allreduce_hook(hook):
    """hook -> hook that runs ``hook`` first and the all-group aggregation after it, as in
    the reference (same misspelt name). Nothing blocks: the returned Future is complete as
    soon as this VSW's bucket has been handed to the GPU's LocalBucketSync."""
    def hook_with_allreduce(state, bucket):
        future_work = hook(state, bucket)
        out = torch.futures.Future()

        def allgroup_allreduce(fut):
            try:
                fut.value()
                idx = bucket_index(bucket)
                want = idx in state._stat_buckets
                state._stat_buckets.discard(idx)

                def stash(stats):
                    if want and stats is not None:
                        state.grad_placeholder.append(stats)

                inner = iidp_allreduce_hook(state, bucket, want_stats=want, on_done=stash)
            except Exception as exc:
                out.set_exception(exc)
                return

            def finish(done):
                try:
                    done.value()
                    out.set_result(bucket_value(bucket, bucket_tensor(bucket)))
                except Exception as exc:
                    out.set_exception(exc)

            inner.add_done_callback(finish)

        future_work.add_done_callback(allgroup_allreduce)
        return out
    return hook_with_allreduce


def cosine_similarity_from_placeholder(grad_placeholder, eps=1e-8):
    """cos(g_A, g_B) over every bucket stashed this step; the counterpart of
    JABASTrainer._compute_cosine_similarity (jabas/train/trainer.py:470-483) without the
    cat / all_gather of two model-sized vectors. Returns a Python float."""
    if not grad_placeholder:
        raise ValueError("no bucket statistics were stashed in this step")
    rows = torch.stack([s.row for s in grad_placeholder])
    return sync.cosine_from_stats(rows, eps)
