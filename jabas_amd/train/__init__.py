from .trainer import VSWSyncTrainer, create_optimizer_hook

__all__ = ["VSWSyncTrainer", "create_optimizer_hook"]
