"""Linear with ``skip_bias_add`` (reference: ``oslo/torch/nn/modules/linear.py:12-35``):
the GEMM itself stays torch's; with ``skip_bias_add=True`` the bias is returned
next to the product so a fused kernel downstream can apply it."""
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor


class Linear(nn.Linear):
    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = True,
        dtype: Optional[torch.dtype] = None,
        skip_bias_add: bool = False,
        device: torch.device = None,
    ):
        super().__init__(in_features, out_features, bias=bias, device=device, dtype=dtype)
        self.skip_bias_add = skip_bias_add

    def forward(self, input: Tensor) -> Union[Tensor, Tuple[Tensor, Tensor]]:
        if self.skip_bias_add:
            return F.linear(input, self.weight), self.bias
        return F.linear(input, self.weight, self.bias)
