"""Batch-size rule and LR modifier on the CPU (restated from jabas/train/trainer.py:649-655,680-718)."""
import math

import pytest

from jabas_amd.train.adaptive import AdaptiveBatchController


def test_low_similarity_grows_and_high_similarity_shrinks_by_the_adjust_rate():
    c = AdaptiveBatchController(128, 32, similarity_target=0.5, adjust_rate=0.1)
    assert c.candidate(0.2) == pytest.approx(128 * 1.1)
    assert c.candidate(0.9) == pytest.approx(128 * 0.9)
    assert c.candidate(0.5) == 128
    one = AdaptiveBatchController(1, 1, 0.5)
    assert one.candidate(0.9) == 1                                # "and self.global_batch_size > 1"


def test_bounds_clamp_the_candidate():
    c = AdaptiveBatchController(128, 32, 0.5, lower_bound=128, upper_bound=128)
    assert c.candidate(0.0) == 128 and c.candidate(1.0) == 128
    workers, mod = c.update(0.0)
    assert workers == 4 and mod == 1.0


def test_placement_keeps_whole_local_batches_and_moves_at_least_one_worker():
    c = AdaptiveBatchController(128, 32, 0.5, adjust_rate=0.1)
    workers, mod = c.update(0.1)                                  # 140.8 -> rounds to 4 -> forced to 5
    assert workers == 5 and c.global_batch_size == 160
    assert mod == pytest.approx(math.sqrt(160 / 128))
    workers, _ = c.update(0.9)                                    # 144 -> 4.5 -> 5 -> must shrink: 4
    assert workers == 4 and c.global_batch_size == 128
    for _ in range(10):
        workers, _ = c.update(0.99)
    assert workers == 1 and c.global_batch_size == 32             # never below one worker
    c2 = AdaptiveBatchController(224, 32, 0.5, max_workers=8)
    for _ in range(5):
        workers, _ = c2.update(-1.0)
    assert workers == 8                                           # at most what one launch aggregates


def test_lr_modifier_uses_the_larger_of_original_and_lower_bound():
    c = AdaptiveBatchController(64, 32, 0.5, lower_bound=128, original_batch_size=64, upper_bound=512)
    workers, mod = c.update(0.0)
    assert c.global_batch_size == workers * 32
    assert mod == pytest.approx(math.sqrt(c.global_batch_size / 128))
    assert c.trajectory[-1][1] == c.global_batch_size


def test_rejects_a_global_size_that_is_not_a_multiple_of_the_local_size():
    with pytest.raises(ValueError):
        AdaptiveBatchController(100, 32, 0.5)
