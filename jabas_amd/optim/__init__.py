from .shard import ShardSGD, ShardAdam, ShardAdamW

__all__ = ["ShardSGD", "ShardAdam", "ShardAdamW"]
