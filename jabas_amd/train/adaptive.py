"""Host-side consumer of the fused statistics: the similarity-based batch-size rule and the
square-root learning-rate modifier.

Restates jabas/train/trainer.py:702-718 (``_adjust_adaptive_global_batch_size``: SimiGrad
Algorithm 1 step 2 -- cos < target grows the global batch size by ``batch_size_adjust_rate``,
cos > target shrinks it), :649-655 (clamping to the configured bounds) and :680-700
(``_scale_lr`` / ``_adjust_adaptive_lr``: modifier = sqrt(new GBS / initial GBS), multiplied
into every group's lr before compute and divided out after step; here it travels as the
``lr_scale`` of the fused launch instead).

The reference then asks IIDP's dynamic-programming solver for a placement that realises
the candidate size with whole local batches (``solve_placement``, un-vendored). On one GPU
the placement is simply the number of VSWs: the candidate is rounded to the nearest
multiple of the local batch size, moving at least one worker in the direction of the
change and staying within 1..max_workers. That rounding is this build's choice.
"""
import math


class AdaptiveBatchController:
    def __init__(self, global_batch_size, local_batch_size, similarity_target, adjust_rate=0.1,
                 lower_bound=None, upper_bound=None, original_batch_size=None, max_workers=8):
        if global_batch_size % local_batch_size:
            raise ValueError("global batch size must be a multiple of the local batch size")
        self.global_batch_size = global_batch_size
        self.local_batch_size = local_batch_size
        self.similarity_target = similarity_target
        self.adjust_rate = adjust_rate
        self.lower_bound, self.upper_bound = lower_bound, upper_bound
        self.original_batch_size = original_batch_size or global_batch_size
        self.max_workers = max_workers
        self.global_lr_modifier = 1.0
        self.trajectory = []

    @property
    def num_workers(self):
        return self.global_batch_size // self.local_batch_size

    def candidate(self, cos):
        """Target size by the similarity rule, clamped to the bounds (may be fractional)."""
        gbs = self.global_batch_size
        if cos < self.similarity_target:
            new = gbs * (1 + self.adjust_rate)
        elif cos > self.similarity_target and gbs > 1:
            new = gbs * (1 - self.adjust_rate)
        else:
            new = gbs
        if self.upper_bound is not None:
            new = min(new, self.upper_bound)
        if self.lower_bound is not None:
            new = max(new, self.lower_bound)
        return new

    def place(self, candidate):
        """Whole number of local batches realising the candidate on this GPU."""
        cur = self.num_workers
        if candidate == self.global_batch_size:
            return cur
        workers = int(math.floor(candidate / self.local_batch_size + 0.5))
        if candidate > self.global_batch_size:
            workers = max(workers, cur + 1)
        else:
            workers = min(workers, cur - 1)
        workers = max(1, min(self.max_workers, workers))
        for bound, clamp in ((self.upper_bound, min), (self.lower_bound, max)):
            if bound is not None:
                lim = bound // self.local_batch_size if clamp is min else -(-bound // self.local_batch_size)
                workers = clamp(workers, max(1, lim))
        return workers

    def update(self, cos, step=None):
        """Applies the rule for one statistic step. Returns (new number of workers, lr modifier)."""
        workers = self.place(self.candidate(float(cos)))
        self.global_batch_size = workers * self.local_batch_size
        initial = self.original_batch_size
        if self.lower_bound is not None:
            initial = max(initial, self.lower_bound)
        self.global_lr_modifier = math.sqrt(self.global_batch_size / initial)
        self.trajectory.append([step, self.global_batch_size])
        return workers, self.global_lr_modifier
