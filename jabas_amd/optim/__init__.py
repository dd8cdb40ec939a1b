from .shard import ShardSGD, ShardAdam, ShardAdamW, ShardGNMTAdam

__all__ = ["ShardSGD", "ShardAdam", "ShardAdamW", "ShardGNMTAdam"]
