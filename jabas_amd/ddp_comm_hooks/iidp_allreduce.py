"""IIDPState and iidp_allreduce_hook for one GPU.

Stand in for iidp.ddp_comm_hooks.iidp_allreduce (un-vendored IIDP submodule; call sites
jabas/ddp_comm_hooks/similarity_allreduce.py:5,10,42 and jabas/train/trainer.py:454-458).
In the reference the hook all-reduces the main VSW's bucket over the world and divides by
``total_num_decoupled_workers``. On one GPU the world is the K local VSWs: the hook
publishes VSW 0's bucket to the LocalBucketSync, and the fused kernel writes the
batch-weighted aggregate (the weights already carry the division) back into that bucket.
"""
from .default_hooks import bucket_tensor, bucket_value, bucket_index, completed, installed_local


class IIDPState:
    def __init__(self, process_group, total_num_decoupled_workers):
        self.process_group = process_group
        self.total_num_decoupled_workers = total_num_decoupled_workers
        self.local = None            # LocalBucketSync of this GPU, see attach_local()
        self.vsw_index = 0

    def attach_local(self, local):
        """Binds the GPU's LocalBucketSync; its K must account for every local VSW. A state nobody
        attached (the reference builds its states without any handle to IIDP's local machinery,
        jabas/train/trainer.py:452-458) takes the meeting point installed for the bucket's device at
        its first hook call."""
        self.local = local
        return self


def iidp_allreduce_hook(state, bucket, want_stats=False, on_done=None):
    tensor = bucket_tensor(bucket)
    value = bucket_value(bucket, tensor)
    local = getattr(state, "local", None)
    if local is None:
        local = installed_local(tensor)
        if local is not None:
            state.local = local
    if local is None:
        if state.total_num_decoupled_workers != 1:
            raise RuntimeError(
                "iidp_allreduce_hook: no LocalBucketSync attached to the state but "
                f"{state.total_num_decoupled_workers} workers declared; this build has no collectives")
        if on_done is not None:
            on_done(None)
        return completed(value)
    return local.publish(0, bucket_index(bucket), tensor, want_stats=want_stats, on_done=on_done, value=value,
                         bucket=bucket)
