"""Flat bucket layout of a gradient set.

``bucket_assignment`` restates DDP's greedy size-capped bucketing
(``torch.distributed._compute_bucket_assignment_by_size`` as driven by
torch/nn/parallel/distributed.py: a bucket is closed as soon as its size reaches the
current cap; the first cap is 1 MiB, every later one 25 MiB) applied in gradient-ready
order, which for the reference's models is the reverse of the registration order. The
reference records the result for ResNet-50 in
examples/resnet50/quickstart/bucket_profile_data/resnet50_bucket_size_profile.json.

``FlatLayout`` places the buckets back to back in one arena (bucket starts aligned to
256 bytes for fp32 and bf16 alike), tensors packed inside a bucket exactly as DDP packs
them, and derives for every bucket the list of parameter-group changes the kernels need.
"""
from collections import namedtuple

MiB = 1024 * 1024
BUCKET_ALIGN_ELEMS = 128          # 512 B of fp32 / 256 B of bf16

Bucket = namedtuple("Bucket", "index param_ids offset numel bounds")


def bucket_assignment(numels, elem_bytes=4, caps=(1 * MiB, 25 * MiB), reverse=True):
    """Returns buckets as lists of tensor indices, in the order the buckets fill up."""
    order = range(len(numels) - 1, -1, -1) if reverse else range(len(numels))
    buckets, cur, size, cap_i = [], [], 0, 0
    for i in order:
        cur.append(i)
        size += numels[i] * elem_bytes
        if size >= caps[min(cap_i, len(caps) - 1)]:
            buckets.append(cur)
            cur, size = [], 0
            cap_i += 1
    if cur:
        buckets.append(cur)
    return buckets


def _round_up(x, m):
    return (x + m - 1) // m * m


class FlatLayout:
    """Arena offsets for a list of ``ParamSpec(name, numel, group)``.

    ``per_tensor_spans`` = True makes every tensor its own span (the worst case for
    launch overhead); otherwise one span per bucket.
    """

    def __init__(self, specs, caps=(1 * MiB, 25 * MiB), elem_bytes=4, per_tensor_spans=False):
        self.specs = list(specs)
        numels = [s.numel for s in self.specs]
        assignment = bucket_assignment(numels, elem_bytes=elem_bytes, caps=caps)
        self.param_offset = [None] * len(self.specs)
        self.param_bucket = [None] * len(self.specs)
        self.buckets = []
        off = 0
        for bi, ids in enumerate(assignment):
            off = _round_up(off, BUCKET_ALIGN_ELEMS)
            start = off
            bounds = []
            for i in ids:
                self.param_offset[i] = off
                self.param_bucket[i] = bi
                g = self.specs[i].group
                if numels[i] and (not bounds or bounds[-1][1] != g):
                    bounds.append((off - start, g))
                off += numels[i]
            self.buckets.append(Bucket(bi, tuple(ids), start, off - start, tuple(bounds)))
        self.total = _round_up(off, BUCKET_ALIGN_ELEMS)
        self.numel = sum(numels)
        self.n_groups = 1 + max([s.group for s in self.specs], default=0)
        if per_tensor_spans:
            self.spans = [(self.param_offset[i], numels[i], ((0, self.specs[i].group),), self.param_bucket[i])
                          for b in self.buckets for i in b.param_ids]
        else:
            self.spans = [(b.offset, b.numel, b.bounds, b.index) for b in self.buckets]

    def bucket_sizes_mb(self, elem_bytes=4):
        return [b.numel * elem_bytes / MiB for b in self.buckets]
