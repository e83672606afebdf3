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
import warnings

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

    ``forward(input, mask)``: ``input`` is ``[b, np, sq, sk]``; ``mask`` is None,
    a boolean tensor with True = masked out, or a floating-point tensor, which
    is an *additive* term: ``softmax(scale * input + mask)``, the form in which
    the reference's models pass their masks and biases (``(1 - m) * -10000`` of
    ``modeling_bert.py:298-306`` and ``modeling_gpt2.py:573-581``, the
    ``finfo.min`` fill of ``models/bart/modeling_bart.py:123-136``, the position
    bias of ``models/t5/modeling_t5.py:508-514``).  Either kind broadcasts
    against the input (up to four dimensions, each leading one 1 or full); the
    fused kernels take a boolean ``[b or 1, 1, sq or 1, sk]`` mask as it is and
    turn any other boolean mask (one per head) into an additive term.
    With the causal type key ``j`` of query ``i`` is hidden when
    ``j > i + (sk - sq)``, whether or not a mask is given: a key-padding mask
    or an additive term then combines with the diagonal in one kernel (the
    loads still stop at the diagonal), which is what a causal model applies to
    a padded batch (``modeling_gpt2.py:126-136``).  When a GPU input cannot
    take the fused kernels the torch chain runs instead and a warning names
    the reason once.
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
        reason = self._unfused_reason(mask, *input.size(), input=input)
        if reason is None:
            return self.forward_fused_softmax(input, mask)
        if input.is_cuda and self.scaled_masked_softmax_fusion:
            self._warn_unfused(reason)
        return self.forward_torch_softmax(input, mask)

    _warned = set()

    def _warn_unfused(self, reason):
        """One warning per reason: a caller who asked for the fused kernels on
        the GPU learns that the torch chain runs instead."""
        if reason not in FusedScaleMaskSoftmax._warned:
            FusedScaleMaskSoftmax._warned.add(reason)
            warnings.warn(
                "FusedScaleMaskSoftmax runs the unfused torch chain: %s" % reason,
                RuntimeWarning, stacklevel=3,
            )

    @staticmethod
    def _broadcasts(mask, b, np, sq, sk):
        if mask.dim() > 4:
            return False
        shape = (1,) * (4 - mask.dim()) + tuple(mask.shape)
        return all(m in (1, full) for m, full in zip(shape, (b, np, sq, sk)))

    def _unfused_reason(self, mask, b, np, sq, sk, input=None):
        """None when the fused kernels take the call, else why they do not."""
        if not self.scaled_masked_softmax_fusion:
            return "scaled_masked_softmax_fusion is off"
        if input is not None:
            if not input.is_cuda:
                return "the input is not on the GPU"
            if input.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                return "input dtype %s (float16, bfloat16 and float32 are fused)" % input.dtype
        if mask is not None:
            if input is not None and mask.device != input.device:
                return "the mask is on %s, the input on %s" % (mask.device, input.device)
            if mask.is_complex() or not self._broadcasts(mask, b, np, sq, sk):
                return "a mask of size %s does not broadcast to [%d, %d, %d, %d]" % (
                    list(mask.shape), b, np, sq, sk)
        if b * np * sq == 0 or sk == 0:
            return "empty input"
        return None

    def is_kernel_available(self, mask, b, np, sq, sk, input=None):
        return self._unfused_reason(mask, b, np, sq, sk, input=input) is None

    @staticmethod
    def _is_key_mask(mask, b, sq, sk):
        """A boolean mask of the shape the mask kernels read directly."""
        return (mask.dim() == 4 and mask.size(1) == 1 and mask.size(3) == sk
                and mask.size(0) in (1, b) and mask.size(2) in (1, sq))

    def forward_fused_softmax(self, input, mask):
        b, np, sq, sk = input.size()
        scale = self.scale if self.scale is not None else 1.0
        p, training = self.attn_dropout, self.training
        causal = self.attn_mask_type == AttnMaskType.causal
        if mask is None:
            if causal:
                probs = onn_f.scaled_upper_triang_masked_softmax_dropout(
                    input.reshape(-1, sq, sk), scale, p, training
                )
                return probs.view(b, np, sq, sk)
            mask = torch.zeros(1, 1, 1, sk, dtype=torch.bool, device=input.device)
        if mask.is_floating_point():
            return onn_f.scaled_bias_softmax_dropout(input, mask, scale, p, training, causal=causal)
        if mask.dtype != torch.bool and mask.dtype != torch.uint8:
            mask = mask != 0
        if self._is_key_mask(mask, b, sq, sk):
            return onn_f.scaled_masked_softmax_dropout(input, mask, scale, p, training, causal=causal)
        # any other boolean mask (one per head): as an additive term whose fill
        # absorbs the logit, so that a row without a visible key is uniform as
        # with the mask kernels; float32 next to float16 scores, whose own lowest
        # value would not
        term_dtype = torch.float32 if input.dtype == torch.float16 else input.dtype
        term = torch.zeros(mask.shape, dtype=term_dtype, device=input.device).masked_fill_(
            mask.bool(), torch.finfo(term_dtype).min
        )
        return onn_f.scaled_bias_softmax_dropout(input, term, scale, p, training, causal=causal)

    def forward_torch_softmax(self, input, mask):
        orig_dtype = input.dtype
        if self.input_in_float16 and self.softmax_in_fp32:
            input = input.float()
        if self.scale is not None:
            input = input * self.scale
        if mask is not None and mask.is_floating_point():
            # an additive term (modeling_bert.py:298-306)
            input = input + mask.to(input.dtype)
            mask = None
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
