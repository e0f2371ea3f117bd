"""Optimizers (nabla/nn/optim/__init__.py)."""
from .functional import adamw_step, sgd_step, sgd_update
from .optimizer import SGD, AdamW, Optimizer, adamw_init, adamw_update

__all__ = ["Optimizer", "SGD", "AdamW", "sgd_step", "sgd_update", "adamw_step", "adamw_init",
           "adamw_update"]
