"""The reference's unfused torch chain for each op, run on CPU tensors.

Test infrastructure only.  Written from the reference's sources (file:line
cited per function; paths relative to EleutherAI/oslo); nothing of the
reference is imported.  These functions are "the reference CPU path": parity
tests compare the HIP kernels with them on identical seeded inputs, and
``bench.py`` times them as the CPU baseline.  Each returns the forward output;
gradients come from torch autograd, as they do in the reference.
"""
import torch
import torch.nn.functional as F


def causal_softmax(x, scale):
    """x: [..., sq, sk].  oslo/transformers/models/gpt2/modeling_gpt2.py:116-138:
    scale, torch.where(causal, w, -1e4), softmax(dim=-1)."""
    sq, sk = x.shape[-2], x.shape[-1]
    w = x * scale
    causal = torch.tril(torch.ones(sk, sk, dtype=torch.bool))[sk - sq:sk, :sk]
    masked_bias = torch.tensor(-1e4, dtype=w.dtype)
    w = torch.where(causal, w, masked_bias)
    return F.softmax(w, dim=-1)


def padding_softmax(x, key_padding, scale):
    """x: [b, np, sq, sk]; key_padding: bool [b, sk], True = padded key.

    oslo/transformers/models/bert/modeling_bert.py:298-306 (scores * scale +
    attention_mask, softmax) with the additive mask built as
    (1 - attend) * -10000 in the scores' dtype (modeling_gpt2.py:573-581).
    """
    attend = (~key_padding).to(x.dtype)[:, None, None, :]
    additive = (1.0 - attend) * -10000.0
    scores = x * scale
    scores = scores + additive
    return F.softmax(scores, dim=-1)


def layer_norm(x, gamma, beta, eps):
    """oslo/torch/nn/modules/layer_norm.py:452-455 (CPU branch of FusedLayerNorm)."""
    return F.layer_norm(x, (x.shape[-1],), gamma, beta, eps)


def rms_norm(x, gamma, eps):
    """oslo/torch/nn/modules/layer_norm.py:17-30 (manual_rms_norm)."""
    variance = x.to(torch.float32).pow(2).mean(-1, keepdim=True)
    y = x * torch.rsqrt(variance + eps)
    if gamma is None:
        return y
    if gamma.dtype in (torch.float16, torch.bfloat16):
        y = y.to(gamma.dtype)
    return gamma * y


def bias_gelu(x, bias):
    """oslo/torch/nn/modules/functional.py:37-40, eager (TorchScript fusion is
    a no-op on current torch); backward by autograd equals :43-50."""
    u = x + bias if bias is not None else x
    return u * 0.5 * (1.0 + torch.tanh(0.79788456 * u * (1 + 0.044715 * u * u)))


def bias_gelu_grad(g, x, bias):
    """oslo/torch/nn/modules/functional.py:43-50 (explicit derivative)."""
    u = x + bias if bias is not None else x
    tanh_out = torch.tanh(0.79788456 * u * (1 + 0.044715 * u * u))
    ff = 0.5 * u * (
        (1 - tanh_out * tanh_out) * (0.79788456 + 0.1070322243 * u * u)
    ) + 0.5 * (1 + tanh_out)
    return ff * g


def bias_dropout_add(x, bias, residual, p, training, keep=None):
    """oslo/torch/nn/modules/functional.py:295-298 (F.dropout(x + bias)) then
    the caller's residual add (modeling_gpt2.py:369, 396).

    With `keep` given (a 0/1 tensor), that mask replaces torch's own draw so the
    result is comparable with a kernel that used the same mask: the ops are
    those F.dropout performs, (x + bias) * keep * (1 / (1 - p)).
    """
    y = x + bias if bias is not None else x
    if keep is None:
        y = F.dropout(y, p=p, training=training)
    elif training and p > 0.0:
        y = y * (keep.to(y.dtype) * (1.0 / (1.0 - p)))
    return y + residual if residual is not None else y
