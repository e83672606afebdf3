"""FusedBiasDropout module (reference: ``oslo/torch/nn/modules/dropout.py:9-11``)."""
import torch
from torch.nn.modules.dropout import _DropoutNd

from oslo_amd.torch.nn.modules.functional import (
    fused_bias_dropout,
    fused_bias_dropout_add,
)


class FusedBiasDropout(_DropoutNd):
    """``dropout(input + bias)``; with ``residual`` given, ``+ residual`` is
    folded into the same kernel (the reference's callers add it afterwards,
    ``modeling_gpt2.py:300, 369``)."""

    def forward(
        self, input: torch.Tensor, bias: torch.Tensor, residual: torch.Tensor = None
    ) -> torch.Tensor:
        if residual is None:
            return fused_bias_dropout(input, bias, self.p, self.training, self.inplace)
        return fused_bias_dropout_add(
            input, bias, residual, self.p, self.training, self.inplace
        )
