"""Public names of the fused non-GEMM transformer ops, mirroring the subset of
the reference's ``oslo/torch/nn/__init__.py:1-53`` that lies on that path, plus
``FusedScaleMaskSoftmax`` (only stubbed in the reference)."""
from oslo_amd.torch.nn.modules.conv import Conv1D
from oslo_amd.torch.nn.modules.dropout import FusedBiasDropout
from oslo_amd.torch.nn.modules.functional import (
    fused_bias_dropout,
    fused_bias_dropout_add,
    fused_bias_dropout_add_layer_norm,
    fused_bias_dropout_add_rms_norm,
    fused_bias_gelu,
    fused_gelu,
    fused_layer_norm,
    fused_layer_norm_affine,
    fused_rms_norm,
    fused_rms_norm_affine,
    mixed_dtype_fused_layer_norm_affine,
    mixed_dtype_fused_rms_norm_affine,
    scaled_bias_softmax,
    scaled_bias_softmax_dropout,
    scaled_masked_softmax,
    scaled_masked_softmax_dropout,
    scaled_upper_triang_masked_softmax,
    scaled_upper_triang_masked_softmax_dropout,
)
from oslo_amd.torch.nn.modules.layer_norm import (
    FusedLayerNorm,
    FusedRMSNorm,
    MixedFusedLayerNorm,
    MixedFusedRMSNorm,
)
from oslo_amd.torch.nn.modules.linear import Linear
from oslo_amd.torch.nn.modules.residual_norm import (
    FusedBiasDropoutAddLayerNorm,
    FusedBiasDropoutAddRMSNorm,
)
from oslo_amd.torch.nn.modules.softmax import (
    AttnMaskType,
    FusedScaleMaskSoftmax,
    attention_mask_func,
)

__all__ = [
    "AttnMaskType",
    "Conv1D",
    "FusedBiasDropout",
    "FusedBiasDropoutAddLayerNorm",
    "FusedBiasDropoutAddRMSNorm",
    "FusedLayerNorm",
    "FusedRMSNorm",
    "FusedScaleMaskSoftmax",
    "Linear",
    "MixedFusedLayerNorm",
    "MixedFusedRMSNorm",
    "attention_mask_func",
    "fused_bias_dropout",
    "fused_bias_dropout_add",
    "fused_bias_dropout_add_layer_norm",
    "fused_bias_dropout_add_rms_norm",
    "fused_bias_gelu",
    "fused_gelu",
    "fused_layer_norm",
    "fused_layer_norm_affine",
    "fused_rms_norm",
    "fused_rms_norm_affine",
    "mixed_dtype_fused_layer_norm_affine",
    "mixed_dtype_fused_rms_norm_affine",
    "scaled_bias_softmax",
    "scaled_bias_softmax_dropout",
    "scaled_masked_softmax",
    "scaled_masked_softmax_dropout",
    "scaled_upper_triang_masked_softmax",
    "scaled_upper_triang_masked_softmax_dropout",
]
