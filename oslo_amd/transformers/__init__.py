"""Model-level helpers that put the fused ops into existing models, mirroring
``oslo/transformers/kernel_fusion_utils.py`` of the reference."""
from oslo_amd.transformers.kernel_fusion_utils import (
    fuse_all,
    fused_attention_forward,
    fused_bias_dropout_add_layer_norm,
    fused_bias_gelu,
    fused_layer_norm,
    fused_pre_ln_block,
    fused_rms_norm,
    fused_scale_mask_softmax,
    register_fused_attention,
)

__all__ = [
    "fuse_all",
    "fused_attention_forward",
    "fused_bias_dropout_add_layer_norm",
    "fused_bias_gelu",
    "fused_layer_norm",
    "fused_pre_ln_block",
    "fused_rms_norm",
    "fused_scale_mask_softmax",
    "register_fused_attention",
]
