"""Module swaps that route a model through the fused kernels.

The reference swaps ``T5LayerNorm`` for ``FusedRMSNorm`` by rewriting the
module's class in place (``oslo/transformers/kernel_fusion_utils.py:71-87``);
``fused_rms_norm`` / ``fused_layer_norm`` do the same here.  The reference's
attention blocks run scale -> mask -> softmax -> dropout unfused
(``oslo/transformers/models/gpt2/modeling_gpt2.py:113-142``);
``fused_scale_mask_softmax`` routes a Hugging Face model's attention through
``FusedScaleMaskSoftmax`` (softmax and attention dropout in one kernel) by
registering an attention function with the library's attention interface.
The reference's post-LN output blocks chain ``FusedBiasDropout``, the residual
add and ``nn.LayerNorm`` (``oslo/transformers/models/bert/modeling_bert.py:337-346,
440-449``); ``fused_bias_dropout_add_layer_norm`` folds the three into the
one-kernel op.
"""
import inspect
import warnings

import torch
import torch.nn as nn

from oslo_amd.torch.nn.modules import functional as onn_f
from oslo_amd.torch.nn.modules.layer_norm import FusedLayerNorm, FusedRMSNorm

ATTENTION_NAME = "oslo_fused_softmax"


def _is_rms_norm(module):
    """T5LayerNorm and its descendants (LlamaRMSNorm, ...): a ``weight`` vector,
    a ``variance_epsilon`` and no bias."""
    return (
        hasattr(module, "variance_epsilon")
        and isinstance(getattr(module, "weight", None), nn.Parameter)
        and module.weight.dim() == 1
        and getattr(module, "bias", None) is None
        and not isinstance(module, (FusedRMSNorm, FusedLayerNorm))
    )


def fused_rms_norm(model):
    """Turns every RMS-norm module of ``model`` into a ``FusedRMSNorm`` in place
    (kernel_fusion_utils.py:71-87 of the reference, there for T5 only).
    Returns the number of modules swapped."""
    n = 0
    for module in model.modules():
        if _is_rms_norm(module):
            module.elementwise_affine = True
            module.normalized_shape = module.weight.size()
            module.eps = module.variance_epsilon
            module.__class__ = FusedRMSNorm
            n += 1
    return n


def fused_layer_norm(model):
    """Turns every ``nn.LayerNorm`` of ``model`` into a ``FusedLayerNorm`` in place."""
    n = 0
    for module in model.modules():
        if type(module) is nn.LayerNorm:
            if module.elementwise_affine and module.bias is None:
                continue  # weight without bias: no fused counterpart
            module.__class__ = FusedLayerNorm
            n += 1
    return n


def _is_post_ln_output(module):
    """``dense`` -> ``dropout`` -> ``LayerNorm(. + input_tensor)``: the shape of
    BertSelfOutput / BertOutput (modeling_bert.py:337-346, 440-449) and of their
    copies in the other post-LN encoders."""
    ln = getattr(module, "LayerNorm", None)
    if not (
        isinstance(getattr(module, "dense", None), nn.Linear)
        and isinstance(getattr(module, "dropout", None), nn.Dropout)
        and isinstance(ln, (nn.LayerNorm, FusedLayerNorm))
        and ln.elementwise_affine
        and ln.bias is not None
    ):
        return False
    try:
        names = list(inspect.signature(type(module).forward).parameters)
    except (TypeError, ValueError):
        return False
    return names == ["self", "hidden_states", "input_tensor"]


def _post_ln_output_forward(self, hidden_states, input_tensor):
    # the dense layer's bias travels to the fused op (skip_bias_add of the
    # reference's linear.py:31-35): bias add, dropout, residual add and
    # LayerNorm are one kernel
    ln = self.LayerNorm
    out = nn.functional.linear(hidden_states, self.dense.weight)
    return onn_f.fused_bias_dropout_add_layer_norm(
        out, self.dense.bias, input_tensor, ln.weight, ln.bias, ln.normalized_shape,
        ln.eps, self.dropout.p, self.training,
    )


_POST_LN_CLASSES = {}


def fused_bias_dropout_add_layer_norm(model):
    """Gives every post-LN output block of ``model`` (dense, dropout, residual
    add, LayerNorm) a forward that runs bias add, dropout, residual add and
    LayerNorm in one kernel; the parameters stay where they are.  Returns the
    number of blocks changed."""
    n = 0
    for module in model.modules():
        cls = type(module)
        if cls in _POST_LN_CLASSES.values() or not _is_post_ln_output(module):
            continue
        if cls not in _POST_LN_CLASSES:
            _POST_LN_CLASSES[cls] = type(
                "Fused" + cls.__name__, (cls,), {"forward": _post_ln_output_forward}
            )
        module.__class__ = _POST_LN_CLASSES[cls]
        n += 1
    return n


def _is_tanh_gelu(act):
    """True when ``act`` computes the tanh form of GeLU the fused kernel
    evaluates (functional.py:23-25 of the reference; "gelu_new",
    "gelu_pytorch_tanh", "gelu_fast" in Hugging Face's table), decided by its
    values, not by its name."""
    probe = torch.linspace(-6.0, 6.0, 97)
    try:
        out = act(probe)
    except Exception:
        return False
    want = 0.5 * probe * (1.0 + torch.tanh(0.79788456 * probe * (1.0 + 0.044715 * probe * probe)))
    return (
        isinstance(out, torch.Tensor)
        and out.shape == probe.shape
        and torch.allclose(out.float(), want, atol=2e-6, rtol=0.0)
    )


def _is_erf_gelu(act):
    """True when ``act`` computes the exact form x * Phi(x) ("gelu" in Hugging
    Face's table), decided by its values."""
    probe = torch.linspace(-6.0, 6.0, 97)
    try:
        out = act(probe)
    except Exception:
        return False
    want = 0.5 * probe * (1.0 + torch.erf(probe * 0.7071067811865476))
    return (
        isinstance(out, torch.Tensor)
        and out.shape == probe.shape
        and torch.allclose(out.float(), want, atol=2e-6, rtol=0.0)
    )


def _is_projection(layer):
    # nn.Linear, or transformers' Conv1D (weight stored [in, out], ``nf`` outputs)
    return isinstance(layer, nn.Linear) or (
        hasattr(layer, "nf") and isinstance(getattr(layer, "weight", None), nn.Parameter)
        and layer.weight.dim() == 2
    )


def _project_gelu(layer, x):
    """gelu(x W + b) with the bias add inside the GeLU kernel."""
    out = _project_no_bias(layer, x)
    if layer.bias is None:
        return onn_f.fused_gelu(out)
    return onn_f.fused_bias_gelu(out, layer.bias)


# (up projection, down projection or None, activation): GPT-2 / GPT-Neo MLP,
# GPT-J MLP, GPT-NeoX / Falcon MLP (no dropout of its own), BERT-style
# intermediate block.  A ``dropout`` child after the down projection is optional.
_MLP_SHAPES = (
    ("c_fc", "c_proj", "act"),
    ("fc_in", "fc_out", "act"),
    ("dense_h_to_4h", "dense_4h_to_h", "act"),
    ("dense", None, "intermediate_act_fn"),
)


def _mlp_shape(module, tanh_for_erf=False):
    try:
        names = list(inspect.signature(type(module).forward).parameters)
    except (TypeError, ValueError):
        return None
    if len(names) != 2 or names[0] != "self":  # forward(self, hidden_states) under any name
        return None
    children = dict(module.named_children())
    for up, down, act in _MLP_SHAPES:
        expected = {up} | ({down} if down else set())
        optional = {act} | ({"dropout"} if down else set())
        if not expected <= set(children) or set(children) - expected - optional:
            continue
        if not _is_projection(children[up]) or (down and not _is_projection(children[down])):
            continue
        if "dropout" in children and not isinstance(children["dropout"], nn.Dropout):
            continue
        fn = getattr(module, act, None)
        if callable(fn) and (_is_tanh_gelu(fn) or (tanh_for_erf and _is_erf_gelu(fn))):
            return up, down
    return None


def _mlp_forward(self, hidden_states):
    up, down = self._oslo_mlp_shape
    h = _project_gelu(getattr(self, up), hidden_states)
    if down is None:
        return h
    h = getattr(self, down)(h)
    dropout = getattr(self, "dropout", None)
    return h if dropout is None else dropout(h)


_MLP_CLASSES = {}


def fused_bias_gelu(model, tanh_for_erf=False):
    """Gives every MLP (or BERT-style intermediate) block of ``model`` whose
    activation is the tanh form of GeLU a forward that adds the up projection's
    bias inside the GeLU kernel (the reference's ``fused_bias_gelu`` over a
    ``skip_bias_add`` linear, linear.py:31-35).  A block is changed only if its
    new forward reproduces the old one on a probe input.  Returns the number
    of blocks changed.

    ``tanh_for_erf=True`` also changes the blocks whose activation is the
    exact form x * Phi(x): the reference's models evaluate the tanh form
    whatever the configuration names (``intermediate_act_fn =
    onn.fused_bias_gelu``, modeling_bert.py:426; modeling_electra.py:469-484;
    modeling_albert.py:333-336), which differs from the exact form by at most
    4.8e-4 in absolute value (4.73e-4 near |x| = 2.3).  Off by default: the swap then changes no
    result of the model beyond rounding."""
    n = 0
    for module in model.modules():
        cls = type(module)
        if cls in _MLP_CLASSES.values():
            continue
        shape = _mlp_shape(module, tanh_for_erf)
        if shape is None:
            continue
        if cls not in _MLP_CLASSES:
            _MLP_CLASSES[cls] = type("Fused" + cls.__name__, (cls,), {"forward": _mlp_forward})
        up = getattr(module, shape[0])
        in_features = up.in_features if isinstance(up, nn.Linear) else up.weight.size(0)
        probe = torch.linspace(-2.0, 2.0, 3 * in_features, device=up.weight.device)
        probe = probe.view(3, in_features).to(up.weight.dtype)
        was_training = module.training
        module.eval()
        with torch.no_grad():
            want = module(probe)
            module._oslo_mlp_shape = shape
            module.__class__ = _MLP_CLASSES[cls]
            got = module(probe)
        module.train(was_training)
        tol = 1e-4 if want.dtype == torch.float32 else 3e-2
        if tanh_for_erf:
            tol += 2e-3  # the two forms of GeLU differ by up to 4.8e-4 before the down projection
        scale = want.float().abs().max().item() + 1e-6
        if (got.float() - want.float()).abs().max().item() > tol * scale:
            module.__class__ = cls  # not the chain it looked like: leave it alone
            del module._oslo_mlp_shape
            continue
        n += 1
    return n


def _project_no_bias(layer, x):
    if isinstance(layer, nn.Linear):
        return nn.functional.linear(x, layer.weight)
    return torch.mm(x.reshape(-1, x.size(-1)), layer.weight).view(x.size()[:-1] + (layer.nf,))


def _no_bias_forward(self, x):
    return _project_no_bias(self, x)


def _identity_forward(self, x):
    return x


_HELPER_CLASSES = {}


def _swap_forward(module, suffix, forward):
    """Rewrites the module's class to a subclass with another forward: the
    parameters, buffers and state-dict keys stay what they were."""
    cls = type(module)
    key = (cls, suffix)
    if key not in _HELPER_CLASSES:
        _HELPER_CLASSES[key] = type(cls.__name__ + suffix, (cls,), {"forward": forward})
    module.__class__ = _HELPER_CLASSES[key]
    return cls


def _is_pre_ln_block(module):
    """ln_1 -> attn (c_proj, resid_dropout) -> +residual -> ln_2 -> mlp (c_proj,
    dropout) -> +residual: the GPT-2 block (modeling_gpt2.py:355-400 of the
    reference), without cross-attention."""
    attn, mlp = getattr(module, "attn", None), getattr(module, "mlp", None)
    ln2 = getattr(module, "ln_2", None)
    return (
        attn is not None and mlp is not None
        and isinstance(getattr(module, "ln_1", None), (nn.LayerNorm, FusedLayerNorm))
        and isinstance(ln2, (nn.LayerNorm, FusedLayerNorm))
        and ln2.elementwise_affine and ln2.bias is not None
        and not hasattr(module, "crossattention")
        and _is_projection(getattr(attn, "c_proj", None))
        and isinstance(getattr(attn, "resid_dropout", None), nn.Dropout)
        and _is_projection(getattr(mlp, "c_proj", None))
        and isinstance(getattr(mlp, "dropout", None), nn.Dropout)
        and attn.c_proj.bias is not None and mlp.c_proj.bias is not None
    )


def _pre_ln_block_forward(self, hidden_states, *args, **kwargs):
    # attn and mlp return their raw output projections (bias and dropout
    # switched off inside them); both bias-dropout-residual steps run fused:
    # the first one together with ln_2, its sum carried on as the residual
    if kwargs.get("encoder_hidden_states") is not None:
        raise ValueError("the fused GPT-2 block has no cross-attention")
    attn_out = self.attn(self.ln_1(hidden_states), *args, **kwargs)
    attn_out = attn_out[0] if isinstance(attn_out, tuple) else attn_out
    ln2 = self.ln_2
    normed, summed = onn_f.fused_bias_dropout_add_layer_norm(
        attn_out, self.attn.c_proj.bias, hidden_states, ln2.weight, ln2.bias,
        ln2.normalized_shape, ln2.eps, self.attn.resid_dropout.p, self.training, True,
    )
    mlp_out = self.mlp(normed)
    return onn_f.fused_bias_dropout_add(
        mlp_out, self.mlp.c_proj.bias, summed, self.mlp.dropout.p, self.training
    )


def fused_pre_ln_block(model):
    """Gives every GPT-2 style pre-LN block of ``model`` a forward in which
    ``dropout(attn_out + bias) + residual`` runs inside the LayerNorm kernel of
    ``ln_2`` and ``dropout(mlp_out + bias) + residual`` as one kernel
    (the residual adds of modeling_gpt2.py:369, 396 of the reference folded into
    its ``FusedBiasDropout``).  A block is changed only if the new forward
    reproduces the old one on a probe input.  Returns the number of blocks
    changed."""
    n = 0
    for module in model.modules():
        if getattr(module, "_oslo_pre_ln", False) or not _is_pre_ln_block(module):
            continue
        width = module.ln_2.normalized_shape[0]
        w = module.ln_2.weight
        probe = torch.linspace(-1.5, 1.5, 2 * 5 * width, device=w.device).view(2, 5, width).to(w.dtype)
        was_training = module.training
        module.eval()
        parts = (module, module.attn.c_proj, module.attn.resid_dropout, module.mlp.c_proj,
                 module.mlp.dropout)
        old = None
        try:
            with torch.no_grad():
                want = module(probe)
                want = want[0] if isinstance(want, tuple) else want
                old = [
                    _swap_forward(parts[0], "FusedResiduals", _pre_ln_block_forward),
                    _swap_forward(parts[1], "NoBias", _no_bias_forward),
                    _swap_forward(parts[2], "Off", _identity_forward),
                    _swap_forward(parts[3], "NoBias", _no_bias_forward),
                    _swap_forward(parts[4], "Off", _identity_forward),
                ]
                got = module(probe)
            tol = 1e-4 if want.dtype == torch.float32 else 3e-2
            scale = want.float().abs().max().item() + 1e-6
            ok = got.shape == want.shape and (got.float() - want.float()).abs().max().item() <= tol * scale
        except Exception:
            ok = False
        module.train(was_training)
        if not ok:
            if old:  # not the chain it looked like: put everything back
                for part, cls in zip(parts, old):
                    part.__class__ = cls
            continue
        module._oslo_pre_ln = True
        n += 1
    return n


def _repeat_kv(hidden_states, n_rep):
    if n_rep == 1:
        return hidden_states
    b, kv_heads, s, d = hidden_states.shape
    hidden_states = hidden_states[:, :, None, :, :].expand(b, kv_heads, n_rep, s, d)
    return hidden_states.reshape(b, kv_heads * n_rep, s, d)


def _unfused_probs(scores, scaling, attention_mask, causal, p, training, out_dtype,
                   position_bias=None):
    """The reference's unfused chain: scale, position bias, mask (boolean True =
    attend, or an additive float term), softmax, dropout."""
    sq, sk = scores.shape[-2], scores.shape[-1]
    t = scores * scaling
    if position_bias is not None:
        t = t + position_bias
    if attention_mask is not None:
        if attention_mask.dtype == torch.bool:
            t = t.masked_fill(~attention_mask, -10000.0)
        else:
            t = t + attention_mask
    elif causal:
        hidden = torch.ones(sq, sk, dtype=torch.bool, device=t.device).triu(1 + sk - sq)
        t = t.masked_fill(hidden, -10000.0)
    probs = torch.softmax(t, dim=-1).to(out_dtype)
    return torch.nn.functional.dropout(probs, p=p, training=training)


def _broadcasts_to(t, shape):
    if t.dim() > len(shape):
        return False
    own = (1,) * (len(shape) - t.dim()) + tuple(t.shape)
    return all(m in (1, full) for m, full in zip(own, shape))


def _unfused_reason(attention_mask, position_bias, scores):
    """None when the fused kernels take the call, else why they cannot."""
    if not scores.is_cuda:
        return "the scores are not on the GPU"
    if scores.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        return "scores of dtype %s" % scores.dtype
    for name, t in (("attention mask", attention_mask), ("position bias", position_bias)):
        if t is None:
            continue
        if t.device != scores.device:
            return "the %s is on %s, the scores on %s" % (name, t.device, scores.device)
        if not _broadcasts_to(t, scores.shape):
            return "a %s of size %s does not broadcast to %s" % (
                name, list(t.shape), list(scores.shape))
    if position_bias is not None and not position_bias.is_floating_point():
        return "a position bias of dtype %s" % position_bias.dtype
    return None


_warned = set()


def _warn_unfused(reason):
    """One warning per reason when scores on the GPU take the torch chain."""
    if reason not in _warned:
        _warned.add(reason)
        warnings.warn(
            "fused_attention_forward runs the unfused torch chain: %s" % reason,
            RuntimeWarning, stacklevel=3,
        )


class CausalKeyPaddingMask(torch.Tensor):
    """The boolean ``[b, 1, sq, sk]`` mask ``causal & key_visible`` of a causal
    model on a padded batch, which remembers its key part ``[b, sk]``: the
    attention function then lets the kernel apply the diagonal and read
    ``[b, sk]`` mask bytes instead of ``[b, sq, sk]``.  The pair survives
    ``.to()`` / ``.cuda()`` / ``.cpu()`` (the key part moves along); any other
    operation returns a plain tensor, and a mask that was written to in place
    after it was built no longer counts (its version is checked), so the key
    part can never describe another mask than the one it travels with."""

    @staticmethod
    def wrap(full, key_visible):
        out = full.as_subclass(CausalKeyPaddingMask)
        out._oslo_key_visible = key_visible
        out._oslo_version = full._version
        return out

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        with torch._C.DisableTorchFunctionSubclass():
            out = func(*args, **kwargs)
        if func in (torch.Tensor.to, torch.Tensor.cuda, torch.Tensor.cpu):
            src = args[0]
            kv = key_visible_of(src)
            if (kv is not None and isinstance(out, torch.Tensor) and out is not src
                    and out.dtype == torch.bool and out.shape == src.shape):
                with torch._C.DisableTorchFunctionSubclass():
                    out = CausalKeyPaddingMask.wrap(out, kv.to(out.device))
        return out


def key_visible_of(mask):
    """The key part of a mask built by ``fused_attention_mask`` when it still
    describes the mask (not written to since), else None."""
    if type(mask) is not CausalKeyPaddingMask:
        return None
    d = mask.__dict__
    kv = d.get("_oslo_key_visible")
    with torch._C.DisableTorchFunctionSubclass():
        if kv is None or d.get("_oslo_version") != mask._version:
            return None
    return kv


def fused_attention_forward(module, query, key, value, attention_mask, scaling=None,
                            dropout=0.0, position_bias=None, **kwargs):
    """Attention with the scale -> mask -> softmax -> dropout chain in one kernel.

    Signature and return value of the attention functions of Hugging Face
    transformers (``(module, query, key, value, attention_mask, scaling,
    dropout, **kwargs) -> (attn_output [b, sq, heads, d], attn_weights)``).
    ``attention_mask`` is None (causal when the module is), a boolean tensor
    with True = attend, or a floating-point tensor, which is an additive term
    (the ``(1 - m) * -10000`` masks of
    oslo/transformers/models/bert/modeling_bert.py:298-306 and
    models/gpt2/modeling_gpt2.py:573-581, the ``finfo.min`` masks of
    models/bart/modeling_bart.py:123-136, ALiBi); ``position_bias`` is the
    relative-position bias T5 adds to its scores
    (models/t5/modeling_t5.py:508-514).  Additive terms go to the kernel that
    computes ``softmax(scale * scores + term)``; a boolean
    ``[b or 1, 1, sq or 1, sk]`` mask to the mask kernel; a mask built by
    ``fused_attention_mask`` for a causal model on a padded batch carries its
    key-padding part, and the kernel then applies the diagonal itself and reads
    ``[b, sk]`` mask bytes instead of ``[b, sq, sk]``.  A boolean mask of
    another shape (one per head) and a boolean mask next to a position bias
    become one additive term.  Scores that are not on the GPU take the
    reference's unfused chain; so does a GPU call the kernels cannot take, with
    a warning that names the reason once.
    """
    if scaling is None:
        scaling = query.size(-1) ** -0.5
    n_rep = query.size(1) // key.size(1)
    key = _repeat_kv(key, n_rep)
    value = _repeat_kv(value, n_rep)
    scores = torch.matmul(query, key.transpose(-1, -2))
    b, heads, sq, sk = scores.shape
    p = float(dropout) if module.training else 0.0
    key_visible = None
    if attention_mask is None:
        causal = kwargs.get("is_causal")
        if causal is None:
            causal = getattr(module, "is_causal", True)
        if position_bias is not None and causal and sq == 1:
            causal = False  # one query against its cache: nothing beyond the diagonal
    else:
        causal = False
        key_visible = key_visible_of(attention_mask)
        if attention_mask.dim() == 4 and attention_mask.size(-1) > sk:
            attention_mask = attention_mask[..., :sk]
            key_visible = None
    reason = _unfused_reason(attention_mask, position_bias, scores)
    if reason is not None:
        if scores.is_cuda:
            _warn_unfused(reason)
        probs = _unfused_probs(scores, scaling, attention_mask, causal, p, module.training,
                               value.dtype, position_bias)
    elif position_bias is not None or (attention_mask is not None
                                       and attention_mask.is_floating_point()):
        # additive terms: the position bias, the mask, or their sum (a boolean
        # mask next to a bias becomes a fill that absorbs the logit)
        term, use_diagonal = position_bias, bool(causal)
        if attention_mask is not None:
            if (key_visible is not None and key_visible.dim() == 2
                    and key_visible.size(-1) == sk and key_visible.device == scores.device):
                # causal pattern x key padding: the kernel applies the diagonal
                attention_mask = key_visible.view(key_visible.size(0), 1, 1, sk)
                use_diagonal = True
            if attention_mask.dtype == torch.bool:
                fill_dtype = term.dtype if term.dtype != torch.float16 else torch.float32
                term = term.to(fill_dtype).masked_fill(~attention_mask, torch.finfo(fill_dtype).min)
            elif term is None:
                term = attention_mask
            else:
                term = term + attention_mask
        probs = onn_f.scaled_bias_softmax_dropout(
            scores, term, scaling, p, module.training, causal=use_diagonal
        )
    elif attention_mask is None and causal:
        probs = onn_f.scaled_upper_triang_masked_softmax_dropout(
            scores.reshape(b * heads, sq, sk), scaling, p, module.training
        ).view(b, heads, sq, sk)
    elif (key_visible is not None and key_visible.dim() == 2 and key_visible.size(-1) == sk
          and key_visible.size(0) in (1, b) and key_visible.device == scores.device):
        # causal pattern x key padding: the diagonal is applied by the kernel
        hidden = (~key_visible).view(key_visible.size(0), 1, 1, sk)
        probs = onn_f.scaled_masked_softmax_dropout(
            scores, hidden, scaling, p, module.training, causal=True
        )
    else:
        if attention_mask is None:
            hidden = torch.zeros(1, 1, 1, sk, dtype=torch.bool, device=scores.device)
        elif attention_mask.dtype == torch.bool:
            hidden = ~attention_mask
        else:
            hidden = attention_mask == 0
        while hidden.dim() < 4:
            hidden = hidden.unsqueeze(0)
        if hidden.size(1) == 1 and hidden.size(3) == sk:
            probs = onn_f.scaled_masked_softmax_dropout(
                scores, hidden, scaling, p, module.training
            )
        else:
            # one mask per head (or per key column only): as an additive term
            # whose fill absorbs the logit, so that a row without a visible key
            # is uniform as with the mask kernel
            fill_dtype = scores.dtype if scores.dtype != torch.float16 else torch.float32
            term = torch.zeros(hidden.shape, dtype=fill_dtype, device=scores.device).masked_fill_(
                hidden, torch.finfo(fill_dtype).min
            )
            probs = onn_f.scaled_bias_softmax_dropout(scores, term, scaling, p, module.training)
    attn_output = torch.matmul(probs.to(value.dtype), value).transpose(1, 2).contiguous()
    return attn_output, probs


def fused_attention_mask(batch_size, q_length, kv_length, q_offset=0, kv_offset=0,
                         mask_function=None, attention_mask=None, **kwargs):
    """Mask builder registered with transformers' mask interface next to
    ``fused_attention_forward``: the boolean mask of ``sdpa_mask`` (True =
    attend), which is correct by itself.  When the pattern is the plain causal
    one whose diagonal is the kernel's (key j of query i visible when
    j <= i + (sk - sq)) and a 2-D padding mask is given, the result is a
    ``CausalKeyPaddingMask`` that carries the key-padding part ``[b, sk]`` and
    the attention function lets the kernel apply the diagonal."""
    from transformers import masking_utils as mu

    if mask_function is None:
        mask_function = mu.causal_mask_function
    if attention_mask is not None and attention_mask.dtype != torch.bool:
        attention_mask = attention_mask != 0
    full = mu.sdpa_mask(batch_size, q_length, kv_length, q_offset=q_offset, kv_offset=kv_offset,
                        mask_function=mask_function, attention_mask=attention_mask, **kwargs)
    if (full is not None and full.dtype == torch.bool and attention_mask is not None
            and mask_function is mu.causal_mask_function
            and isinstance(q_offset, int) and isinstance(kv_offset, int)
            and q_offset - kv_offset == kv_length - q_length):
        try:
            kv = mu.prepare_padding_mask(attention_mask, kv_length, kv_offset)
            kv = kv[:, kv_offset:kv_offset + kv_length]
        except Exception:  # noqa: BLE001 - an internal helper: without it the full mask is used
            kv = None
        if kv is not None and kv.dim() == 2 and kv.size(-1) == kv_length and kv.size(0) in (1, batch_size):
            full = CausalKeyPaddingMask.wrap(full, kv.to(device=full.device, dtype=torch.bool))
    return full


def register_fused_attention(name=ATTENTION_NAME):
    """Registers ``fused_attention_forward`` (and its boolean mask builder) with
    transformers' attention interface under ``name``."""
    try:
        from transformers import AttentionInterface
        from transformers.masking_utils import AttentionMaskInterface, sdpa_mask  # noqa: F401
    except ImportError as e:  # older transformers: no pluggable attention
        raise ImportError(
            "fused_scale_mask_softmax needs a transformers version with "
            "AttentionInterface (%s)" % e
        ) from None
    AttentionInterface.register(name, fused_attention_forward)
    AttentionMaskInterface.register(name, fused_attention_mask)
    return name


def fused_scale_mask_softmax(model, name=ATTENTION_NAME):
    """Routes the attention of a Hugging Face ``model`` through the fused
    scale-mask-softmax(-dropout) kernels."""
    register_fused_attention(name)
    if hasattr(model, "set_attn_implementation"):
        model.set_attn_implementation(name)
    else:
        model.config._attn_implementation = name
    # sub-models that hold their own copy of the configuration (the encoder
    # and decoder stacks of T5) are not reached by the call above
    seen = {id(getattr(model, "config", None))}
    for module in model.modules():
        cfg = getattr(module, "config", None)
        if cfg is None or id(cfg) in seen or not hasattr(cfg, "_attn_implementation"):
            continue
        seen.add(id(cfg))
        try:
            cfg._attn_implementation = name
        except (ValueError, AttributeError):
            pass  # a configuration that refuses the name keeps its own attention
    return model


def fuse_all(model, attention=True, tanh_for_erf=False):
    """Applies every swap of this module that fits ``model``; returns how many
    modules each one changed (``attention`` is True/False: the attention
    function is a property of the whole model; ``tanh_for_erf``: see
    ``fused_bias_gelu``)."""
    changed = {
        "fused_pre_ln_block": fused_pre_ln_block(model),
        "fused_bias_dropout_add_layer_norm": fused_bias_dropout_add_layer_norm(model),
        "fused_bias_gelu": fused_bias_gelu(model, tanh_for_erf),
        "fused_layer_norm": fused_layer_norm(model),
        "fused_rms_norm": fused_rms_norm(model),
        "fused_scale_mask_softmax": False,
    }
    if attention and hasattr(model, "config"):
        try:
            fused_scale_mask_softmax(model)
            # (a model without pluggable attention keeps its own implementation)
            changed["fused_scale_mask_softmax"] = (
                getattr(model.config, "_attn_implementation", None) == ATTENTION_NAME
            )
        except (ImportError, ValueError):
            pass  # no pluggable attention in this model / library version
    return changed
