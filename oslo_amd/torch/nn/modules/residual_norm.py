"""Bias + dropout + residual add fused into the LayerNorm / RMSNorm that follows.

The reference's blocks chain three modules here -- ``FusedBiasDropout``, the
residual add and ``nn.LayerNorm``
(``oslo/transformers/models/bert/modeling_bert.py:337-346, 440-449``; pre-LN:
``oslo/transformers/models/gpt2/modeling_gpt2.py:369-393``).  These modules own
the norm's parameters and take the dense layer's ``(out, bias)`` pair
(``skip_bias_add=True``) together with the residual.
"""
import numbers

import torch
from torch.nn import Parameter, init
from torch.nn.modules.dropout import _DropoutNd

from oslo_amd.torch.nn.modules import functional as onn_f


class _FusedBiasDropoutAddNorm(_DropoutNd):
    _rms = False

    def __init__(self, normalized_shape, p=0.0, eps=1e-5, elementwise_affine=True,
                 return_sum=False):
        super().__init__(p=p, inplace=False)
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        self.return_sum = return_sum
        if elementwise_affine:
            self.weight = Parameter(torch.Tensor(*normalized_shape))
            if self._rms:
                self.register_parameter("bias", None)
            else:
                self.bias = Parameter(torch.Tensor(*normalized_shape))
        else:
            self.register_parameter("weight", None)
            self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        if self.elementwise_affine:
            init.ones_(self.weight)
            if self.bias is not None:
                init.zeros_(self.bias)

    def forward(self, input, bias=None, residual=None):
        """``norm(dropout(input + bias) + residual)``; with ``return_sum`` a pair
        ``(normalised, dropout(input + bias) + residual)``."""
        if self._rms:
            return onn_f.fused_bias_dropout_add_rms_norm(
                input, bias, residual, self.weight, self.normalized_shape, self.eps,
                self.p, self.training, self.return_sum,
            )
        return onn_f.fused_bias_dropout_add_layer_norm(
            input, bias, residual, self.weight, self.bias, self.normalized_shape,
            self.eps, self.p, self.training, self.return_sum,
        )

    def extra_repr(self):
        return (
            "{normalized_shape}, p={p}, eps={eps}, "
            "elementwise_affine={elementwise_affine}".format(**self.__dict__)
        )


class FusedBiasDropoutAddLayerNorm(_FusedBiasDropoutAddNorm):
    """``LayerNorm(dropout(input + bias, p) + residual)`` in one kernel."""

    _rms = False


class FusedBiasDropoutAddRMSNorm(_FusedBiasDropoutAddNorm):
    """``RMSNorm(dropout(input + bias, p) + residual)`` in one kernel."""

    _rms = True
