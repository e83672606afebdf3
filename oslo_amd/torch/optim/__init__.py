"""Fused optimizers (``oslo/torch/optim/__init__.py`` of the reference; Adam only)."""
from oslo_amd.torch.optim.fused_adam import FusedAdam

__all__ = ["FusedAdam"]
