"""FusedScaleMaskSoftmax: scale -> mask -> softmax over attention scores.

The reference ships only the pybind shim of this op
(``oslo/torch/_C/csrc/FusedScaleMaskSoftmaxBinder.cpp:39-127``: five entry
points, no kernel and no Python module), and its models run the unfused chain
(``oslo/transformers/models/gpt2/modeling_gpt2.py:116-138``,
``oslo/transformers/models/bert/modeling_bert.py:298-306``).  This module is the
caller that shim was written for: constructor and ``forward(input, mask)`` follow
the Megatron-LM module of the same name, the fused branch calls the HIP kernels
and the unfused branch is the reference's torch chain.  Unlike the shim, fp32
inputs and any sequence length are accepted by the fused branch.
"""
import enum

import torch
import torch.nn as nn

from oslo_amd.torch.nn.modules import functional as onn_f


class AttnMaskType(enum.Enum):
    padding = 1
    causal = 2


def attention_mask_func(attention_scores, attention_mask):
    """Default ``mask_func``: masked positions (True) are filled with -10000."""
    return attention_scores.masked_fill(attention_mask, -10000.0)


class FusedScaleMaskSoftmax(nn.Module):
    """
    Args:
        input_in_fp16: the scores arrive in fp16.
        input_in_bf16: the scores arrive in bf16.
        attn_mask_type: ``AttnMaskType.causal`` or ``AttnMaskType.padding``.
        scaled_masked_softmax_fusion: use the fused kernels when possible.
        mask_func: ``(scores, mask) -> scores`` used by the unfused branch.
        softmax_in_fp32: unfused branch computes the softmax in fp32 (the fused
            kernels always accumulate in fp32).
        scale: factor applied to the scores before masking (None = 1).
        attn_dropout: probability of the dropout the models apply to the
            probabilities right after the softmax
            (``modeling_gpt2.py:142``, ``modeling_bert.py:310``); fused into the
            same kernel while the module is in training mode.  0 (default)
            leaves the module a plain softmax.

    ``forward(input, mask)``: ``input`` is ``[b, np, sq, sk]``; ``mask`` is a
    boolean ``[b or 1, 1, sq or 1, sk]`` tensor with True = masked out, or None.
    With the causal type key ``j`` of query ``i`` is hidden when
    ``j > i + (sk - sq)``, whether or not a mask is given: a key-padding mask
    then combines with the diagonal in one kernel (the loads still stop at the
    diagonal), which is what a causal model applies to a padded batch
    (``modeling_gpt2.py:126-136``).
    """

    def __init__(
        self,
        input_in_fp16=False,
        input_in_bf16=False,
        attn_mask_type=AttnMaskType.padding,
        scaled_masked_softmax_fusion=True,
        mask_func=attention_mask_func,
        softmax_in_fp32=True,
        scale=None,
        attn_dropout=0.0,
    ):
        super().__init__()
        if attn_dropout < 0.0 or attn_dropout > 1.0:
            raise ValueError(
                "dropout probability has to be between 0 and 1, but got {}".format(
                    attn_dropout
                )
            )
        self.attn_dropout = float(attn_dropout)
        self.input_in_fp16 = input_in_fp16
        self.input_in_bf16 = input_in_bf16
        if self.input_in_fp16 and self.input_in_bf16:
            raise ValueError("both fp16 and bf16 flags cannot be active at the same time.")
        self.input_in_float16 = self.input_in_fp16 or self.input_in_bf16
        self.attn_mask_type = attn_mask_type
        self.scaled_masked_softmax_fusion = scaled_masked_softmax_fusion
        self.mask_func = mask_func
        self.softmax_in_fp32 = softmax_in_fp32
        self.scale = scale
        if not (self.scale is None or softmax_in_fp32):
            raise ValueError("softmax should be in fp32 when scaled")

    def forward(self, input, mask):
        if input.dim() != 4:
            raise RuntimeError("expected 4D tensor [b, np, sq, sk]")
        if self.is_kernel_available(mask, *input.size(), input=input):
            return self.forward_fused_softmax(input, mask)
        return self.forward_torch_softmax(input, mask)

    def is_kernel_available(self, mask, b, np, sq, sk, input=None):
        if not self.scaled_masked_softmax_fusion:
            return False
        if input is not None:
            if not input.is_cuda:
                return False
            if input.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                return False
        if mask is not None:
            # the kernels take "masked out or not" per key; an additive float
            # mask (which may carry finite biases) is left to mask_func
            if mask.is_floating_point():
                return False
            if input is not None and mask.device != input.device:
                return False
            if mask.dim() != 4 or mask.size(1) != 1 or mask.size(3) != sk:
                return False
            if mask.size(0) not in (1, b) or mask.size(2) not in (1, sq):
                return False
        return b * np * sq > 0 and sk > 0

    def forward_fused_softmax(self, input, mask):
        b, np, sq, sk = input.size()
        scale = self.scale if self.scale is not None else 1.0
        p, training = self.attn_dropout, self.training
        if self.attn_mask_type == AttnMaskType.causal and mask is None:
            probs = onn_f.scaled_upper_triang_masked_softmax_dropout(
                input.reshape(-1, sq, sk), scale, p, training
            )
            return probs.view(b, np, sq, sk)
        if mask is None:
            mask = torch.zeros(1, 1, 1, sk, dtype=torch.bool, device=input.device)
        causal = self.attn_mask_type == AttnMaskType.causal
        return onn_f.scaled_masked_softmax_dropout(input, mask, scale, p, training, causal=causal)

    def forward_torch_softmax(self, input, mask):
        orig_dtype = input.dtype
        if self.input_in_float16 and self.softmax_in_fp32:
            input = input.float()
        if self.scale is not None:
            input = input * self.scale
        if self.attn_mask_type == AttnMaskType.causal:
            sq, sk = input.size(2), input.size(3)
            causal = torch.ones(sq, sk, dtype=torch.bool, device=input.device).triu(
                diagonal=1 + sk - sq
            )
            causal = causal.view(1, 1, sq, sk)
            mask = causal if mask is None else (mask.bool() | causal)
        mask_output = self.mask_func(input, mask) if mask is not None else input
        probs = torch.nn.Softmax(dim=-1)(mask_output)
        if self.input_in_float16 and self.softmax_in_fp32:
            probs = probs.to(orig_dtype)
        if self.attn_dropout > 0.0:
            probs = torch.nn.functional.dropout(
                probs, p=self.attn_dropout, training=self.training
            )
        return probs

    @staticmethod
    def get_batch_per_block(sq, sk, b, np):
        from oslo_amd.torch._C import get_softmax_kernel

        return get_softmax_kernel().get_batch_per_block(sq, sk, b, np)
