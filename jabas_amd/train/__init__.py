from .trainer import (VSWSyncTrainer, create_optimizer_hook, create_stream_for_optimizer,
                      prepare_overlap_optimizer_with_ddp)

__all__ = ["VSWSyncTrainer", "create_optimizer_hook", "create_stream_for_optimizer",
           "prepare_overlap_optimizer_with_ddp"]
