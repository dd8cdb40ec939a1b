"""Bucket adapters and the hooks every VSW but the first registers.

Stands in for iidp.ddp_comm_hooks.default_hooks (un-vendored IIDP submodule; call sites
jabas/ddp_comm_hooks/similarity_allreduce.py:4,30 and jabas/train/trainer.py:461-468).
Both bucket flavours are accepted: torch 1.8.1's ``_GradBucket`` (``get_tensors()``,
futures carry a list) that the reference targets, and today's ``GradBucket``
(``buffer()``, futures carry a tensor).
"""
import torch
import torch.distributed as dist


def bucket_tensor(bucket):
    if hasattr(bucket, "buffer"):
        return bucket.buffer()
    return bucket.get_tensors()[0]


def bucket_value(bucket, tensor):
    """What a hook's Future must carry for this bucket flavour."""
    return tensor if hasattr(bucket, "buffer") else [tensor]


def bucket_index(bucket):
    for name in ("index", "get_index"):
        fn = getattr(bucket, name, None)
        if callable(fn):
            return int(fn())
    raise AttributeError("bucket object exposes neither index() nor get_index()")


def completed(value):
    fut = torch.futures.Future()
    fut.set_result(value)
    return fut


def _allreduce_sum_fut(group, tensor):
    """Sum of ``tensor`` over ``group`` as a Future of ``[tensor]``. One process (the only
    case this build runs): the sum over one rank is the tensor itself. With an
    initialised multi-rank process group it defers to torch.distributed."""
    if not (dist.is_available() and dist.is_initialized()) or dist.get_world_size(group) == 1:
        return completed([tensor])
    work = dist.all_reduce(tensor, group=group, async_op=True)
    return work.get_future().then(lambda fut: [fut.value()[0] if isinstance(fut.value(), (list, tuple)) else fut.value()])


class VSWPeerState:
    """State a non-main VSW may register with ``dummy_hook`` to name its meeting point and VSW index
    itself. The reference registers ``state=None`` (jabas/train/trainer.py:466-468); ``dummy_hook`` then
    finds both on its own."""

    def __init__(self, local, vsw_index):
        self.local, self.vsw_index = local, vsw_index


def installed_local(tensor):
    """The LocalBucketSync installed for the device ``tensor`` lives on, or None."""
    from ..local_sync import installed
    return installed(tensor.device if tensor.is_cuda else None)


def dummy_hook(state, bucket):
    """The hook of every VSW but the first (jabas/train/trainer.py:461-468, registered with ``state=None``):
    hands the replica's bucket to the GPU's meeting point and returns at once. The meeting point is the one
    installed for the bucket's device (``LocalBucketSync.install``), the VSW index comes from the bucket's
    parameters (``register_replicas``) or from the stream the hook runs on. With no meeting point installed
    (a single VSW, or plain DDP) the hook is the pass-through its name says."""
    tensor = bucket_tensor(bucket)
    local = getattr(state, "local", None) if state is not None else installed_local(tensor)
    if local is None:
        return completed(bucket_value(bucket, tensor))
    k = state.vsw_index if state is not None else local.vsw_of(bucket, tensor)
    return local.publish(k, bucket_index(bucket), tensor, value=bucket_value(bucket, tensor), bucket=bucket)
