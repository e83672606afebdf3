"""Fused optimizers (``oslo/torch/optim/__init__.py`` of the reference): every
class updates all parameters of a group with a few multi-tensor kernel launches."""
from oslo_amd.torch.optim.fused_adagrad import FusedAdagrad
from oslo_amd.torch.optim.fused_adam import FusedAdam
from oslo_amd.torch.optim.fused_lamb import FusedLamb
from oslo_amd.torch.optim.fused_mixed_precision_lamb import FusedMixedPrecisionLamb
from oslo_amd.torch.optim.fused_novograd import FusedNovograd
from oslo_amd.torch.optim.fused_sgd import FusedSGD

__all__ = ["FusedAdam", "FusedAdagrad", "FusedLamb", "FusedMixedPrecisionLamb", "FusedNovograd", "FusedSGD"]
