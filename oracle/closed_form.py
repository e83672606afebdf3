"""numpy restatement of the hot path's arithmetic.  Test infrastructure only.

Every function takes numpy arrays holding the operands' exact values (a bf16
or fp16 tensor is passed as the float32/float64 array of its values), computes
in ``acc`` precision (float64 unless stated) and, where ``out`` names a storage
type, rounds the result to it once at the point where the fused kernel rounds.
File:line citations are into the reference repository (EleutherAI/oslo).

Pinning: the reference holds no numeric vectors, known answers or fixtures for
these ops (its tests compare two of its own paths on unseeded data), so none of
the functions here is pinned by reference-held data.  Each one is pinned
instead by tests/test_oracle_closed_form.py, test_oracle_philox.py,
test_oracle_adam.py and test_oracle_optimizers.py: torch library routines
(torch.optim among them) and torch autograd in float64,
finite differences, invariants (row sums, shift invariance, exact zeros,
orthogonality of the norm gradients), brute force on tiny inputs and the
Random123 known-answer vectors.
"""
import numpy as np

GELU_A = 0.79788456  # oslo/torch/nn/modules/functional.py:25
GELU_B = 0.044715  # functional.py:25
GELU_C = 0.1070322243  # functional.py:32


# ---------------------------------------------------------------------------
# storage-type rounding
# ---------------------------------------------------------------------------
def round_bf16(a):
    """Round-to-nearest-even to bfloat16, returned as float32 values."""
    a32 = np.ascontiguousarray(a, dtype=np.float32)
    u = a32.view(np.uint32).astype(np.uint64)
    bias = ((u >> 16) & 1) + 0x7FFF
    r = ((u + bias) & 0xFFFF0000).astype(np.uint32)
    out = r.view(np.float32).reshape(a32.shape).copy()
    nan = np.isnan(a32)
    if nan.any():
        out[nan] = np.nan
    return out


def round_f16(a):
    """Round-to-nearest-even to float16 by way of float32 (see round_to),
    returned as float32 values."""
    return np.asarray(a, dtype=np.float64).astype(np.float32).astype(np.float16).astype(np.float32)


def round_to(a, out):
    """out in {'f32', 'f16', 'bf16', 'f64'}: value after storing `a` as that type.

    Rounding a float64 value to bf16/fp16 goes through float32 first, as the
    kernels' fp32 arithmetic does; the double rounding differs from direct
    rounding only for values within 2^-29 relative of a tie.
    """
    if out == "f64":
        return np.asarray(a, dtype=np.float64)
    if out == "f32":
        return np.asarray(a, dtype=np.float64).astype(np.float32)
    if out == "f16":
        return round_f16(a)
    if out == "bf16":
        return round_bf16(np.asarray(a, dtype=np.float64).astype(np.float32))
    raise ValueError(out)


def ulp_of(out):
    """Relative spacing (2^-mantissa_bits) of a storage type."""
    return {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7, "f64": 2.0 ** -52}[out]


# ---------------------------------------------------------------------------
# softmax
# ---------------------------------------------------------------------------
def causal_hidden(sq, sk):
    """True where key j is hidden from query i: j > i + (sk - sq).

    The lower-triangular visibility of
    oslo/transformers/models/gpt2/modeling_gpt2.py:126-132 (bias[..., sk-sq:sk, :sk]).
    """
    i = np.arange(sq)[:, None]
    j = np.arange(sk)[None, :]
    return j > i + (sk - sq)


def softmax_masked_fwd(x, hidden, scale, out="f64", acc=np.float64):
    """y = softmax(scale * x) over visible keys; hidden keys get exactly 0; a
    row with no visible key becomes uniform 1/sk.

    modeling_gpt2.py:116-138 (scale, where(causal, w, -1e4), softmax) and
    oslo/transformers/models/bert/modeling_bert.py:298-306 (scale, additive
    mask, softmax): exp(-1e4 - max) underflows to 0 in every storage type, so
    the fill value is the limit "probability 0"; a fully hidden row is
    softmax of a constant = uniform.  `hidden` broadcasts against `x`.
    """
    x = np.asarray(x, dtype=acc)
    hidden = np.broadcast_to(np.asarray(hidden, dtype=bool), x.shape)
    t = np.where(hidden, -np.inf, x * acc(scale))
    m = t.max(axis=-1, keepdims=True)
    empty = np.isneginf(m)
    m = np.where(empty, 0.0, m)
    e = np.exp(t - m)
    s = e.sum(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        y = np.where(empty, acc(1.0) / x.shape[-1], e / np.where(empty, 1.0, s))
    return round_to(y, out)


def softmax_causal_fwd(x, scale, out="f64", acc=np.float64):
    """x: [attn_batches, sq, sk]
    (oslo/torch/_C/csrc/FusedScaleMaskSoftmaxBinder.cpp:76-86)."""
    sq, sk = x.shape[-2], x.shape[-1]
    return softmax_masked_fwd(x, causal_hidden(sq, sk), scale, out, acc)


def softmax_bwd(dy, y, scale, out="f64", acc=np.float64):
    """dx = scale * y * (dy - sum_j dy_j y_j)
    (closed form also held by the reference's LightSeq test,
    oslo/lightseq2/csrc/tests/cuda/test_kernel.py:361-368, there without scale)."""
    dy = np.asarray(dy, dtype=acc)
    y = np.asarray(y, dtype=acc)
    s = (dy * y).sum(axis=-1, keepdims=True)
    return round_to(acc(scale) * (y * (dy - s)), out)


def _dropout_scale(p, acc):
    return acc(np.float32(1.0) / (np.float32(1.0) - np.float32(p))) if p < 1.0 else acc(0.0)


def softmax_dropout_fwd(x, hidden, scale, keep, p, out="f64", acc=np.float64):
    """out = keep * softmax(mask(scale * x)) / (1 - p), rounded once.

    The softmax of modeling_gpt2.py:138 / modeling_bert.py:306 followed by
    attn_dropout (modeling_gpt2.py:142, modeling_bert.py:310), i.e.
    torch.nn.functional.dropout of the probabilities.  `keep` is the 0/1 mask
    over the output (None = keep everything).
    """
    y = softmax_masked_fwd(x, hidden, scale, "f64", acc)
    if keep is not None:
        y = np.where(np.asarray(keep, dtype=bool), y * _dropout_scale(p, acc), 0.0)
    return round_to(y, out)


def softmax_dropout_bwd(dout, x, hidden, scale, keep, p, out="f64", acc=np.float64):
    """dx of out = dropout(softmax(mask(scale * x))) given d(out):
    dp = keep * dout / (1 - p) is the gradient of the probabilities y, then the
    softmax backward dx = scale * y * (dp - sum_k dp_k y_k), with y recomputed
    from x in `acc` precision (the fused backward keeps x, not y)."""
    y = softmax_masked_fwd(x, hidden, scale, "f64", acc)
    dp = np.asarray(dout, dtype=acc)
    if keep is not None:
        dp = np.where(np.asarray(keep, dtype=bool), dp * _dropout_scale(p, acc), 0.0)
    s = (dp * y).sum(axis=-1, keepdims=True)
    return round_to(acc(scale) * (y * (dp - s)), out)


def softmax_bias_fwd(x, bias, scale, causal=False, out="f64", acc=np.float64, sum_f32=True):
    """y = softmax(scale * x + bias): the scores with an additive term, which
    is how the reference's models mask and bias them
    (oslo/transformers/models/bert/modeling_bert.py:298-306: scores / sqrt(d) +
    attention_mask; modeling_gpt2.py:136 with the (1 - m) * -10000 mask of
    :573-581; the finfo.min fill of models/bart/modeling_bart.py:123-136,
    262-284; the position bias of models/t5/modeling_t5.py:508-514).

    `bias` broadcasts against `x`.  With `sum_f32` the sum is rounded to
    float32 once (the fused kernel forms it by one float multiply-add), so
    that a term of -10000 costs the logit the same bits here and there and
    the lowest finite float absorbs the logit altogether; without it the
    function is the plain float64 softmax of the sum.  `causal` hides key j of
    query i for j > i + (sk - sq) (probability exactly 0).  A row of -inf
    sums is NaN, as torch.softmax returns it.
    """
    x = np.asarray(x, dtype=acc)
    with np.errstate(over="ignore", invalid="ignore"):
        t = x * acc(scale) + np.broadcast_to(np.asarray(bias, dtype=acc), x.shape)
        if sum_f32:
            t = t.astype(np.float32).astype(acc)
    if causal:
        t = np.where(causal_hidden(x.shape[-2], x.shape[-1]), -np.inf, t)
    with np.errstate(invalid="ignore"):
        m = t.max(axis=-1, keepdims=True)
        e = np.exp(t - m)  # (-inf) - (-inf) = NaN for a row without a finite sum
        y = e / e.sum(axis=-1, keepdims=True)
    return round_to(y, out)


def softmax_bias_dropout_fwd(x, bias, scale, keep, p, causal=False, out="f64", acc=np.float64):
    """out = keep * softmax(scale * x + bias) / (1 - p), rounded once."""
    y = softmax_bias_fwd(x, bias, scale, causal, "f64", acc)
    if keep is not None:
        y = np.where(np.asarray(keep, dtype=bool), y * _dropout_scale(p, acc), 0.0)
    return round_to(y, out)


def softmax_bias_dropout_bwd(dout, x, bias, scale, keep, p, causal=False, out="f64",
                             acc=np.float64):
    """dx of out = dropout(softmax(scale * x + bias)) given d(out); the
    gradient of the additive term is dx / scale summed over the dimensions it
    broadcasts along."""
    y = softmax_bias_fwd(x, bias, scale, causal, "f64", acc)
    dp = np.asarray(dout, dtype=acc)
    if keep is not None:
        dp = np.where(np.asarray(keep, dtype=bool), dp * _dropout_scale(p, acc), 0.0)
    s = (dp * y).sum(axis=-1, keepdims=True)
    return round_to(acc(scale) * (y * (dp - s)), out)


# ---------------------------------------------------------------------------
# LayerNorm / RMSNorm
# ---------------------------------------------------------------------------
def layer_norm_fwd(x, gamma, beta, eps, out="f64", acc=np.float64):
    """Returns (y, mean, invvar) over the last axis.

    mean / biased variance / invvar = rsqrt(var + eps) as
    oslo/torch/_C/csrc/fused_layer_norm.cu:310-359; y = (x - mean) * invvar
    * gamma + beta evaluated in `acc` and rounded once, which is what
    torch.nn.functional.layer_norm (the reference's CPU path,
    oslo/torch/nn/modules/layer_norm.py:452-455) does for 16-bit tensors.
    """
    x = np.asarray(x, dtype=acc)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    invvar = 1.0 / np.sqrt(var + acc(eps))
    y = (x - mean) * invvar
    if gamma is not None:
        y = y * np.asarray(gamma, dtype=acc) + np.asarray(beta, dtype=acc)
    return round_to(y, out), mean[..., 0], invvar[..., 0]


def layer_norm_bwd(dy, x, mean, invvar, gamma, out_dx="f64", out_param="f64", acc=np.float64):
    """Returns (dx, dgamma, dbeta); fused_layer_norm.cu:594-741 (dx) and
    :458-591 (dgamma = sum dy * xhat, dbeta = sum dy)."""
    dy = np.asarray(dy, dtype=acc)
    x = np.asarray(x, dtype=acc)
    n2 = x.shape[-1]
    mean = np.asarray(mean, dtype=acc)[..., None]
    invvar = np.asarray(invvar, dtype=acc)[..., None]
    xhat = (x - mean) * invvar
    g = 1.0 if gamma is None else np.asarray(gamma, dtype=acc)
    dyg = dy * g
    s1 = dyg.sum(axis=-1, keepdims=True)
    s2 = (dyg * xhat).sum(axis=-1, keepdims=True)
    dx = (n2 * dyg - s1 - xhat * s2) * (invvar / n2)
    if gamma is None:
        return round_to(dx, out_dx), None, None
    flat_dy = dy.reshape(-1, n2)
    flat_xh = xhat.reshape(-1, n2)
    dgamma = (flat_dy * flat_xh).sum(axis=0)
    dbeta = flat_dy.sum(axis=0)
    return round_to(dx, out_dx), round_to(dgamma, out_param), round_to(dbeta, out_param)


def rms_norm_fwd(x, gamma, eps, out="f64", acc=np.float64):
    """Returns (y, invvar).  invvar = rsqrt(mean(x^2) + eps); the normalised
    value is rounded to the output type BEFORE the scale by gamma, then the
    product is rounded again: layer_norm.py:20-30 (manual_rms_norm) and
    fused_layer_norm.cu:338 agree on that order."""
    x = np.asarray(x, dtype=acc)
    invvar = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + acc(eps))
    y = round_to(x * invvar, out)
    if gamma is not None:
        y = round_to(np.asarray(gamma, dtype=acc) * np.asarray(y, dtype=acc), out)
    return y, invvar[..., 0]


def rms_norm_bwd(dy, x, invvar, gamma, out_dx="f64", out_param="f64", acc=np.float64):
    """Returns (dx, dgamma); fused_layer_norm.cu:594-741 with rms_only."""
    dy = np.asarray(dy, dtype=acc)
    x = np.asarray(x, dtype=acc)
    n2 = x.shape[-1]
    invvar = np.asarray(invvar, dtype=acc)[..., None]
    xhat = x * invvar
    g = 1.0 if gamma is None else np.asarray(gamma, dtype=acc)
    dyg = dy * g
    s2 = (dyg * xhat).sum(axis=-1, keepdims=True)
    dx = (n2 * dyg - xhat * s2) * (invvar / n2)
    if gamma is None:
        return round_to(dx, out_dx), None
    dgamma = (dy.reshape(-1, n2) * xhat.reshape(-1, n2)).sum(axis=0)
    return round_to(dx, out_dx), round_to(dgamma, out_param)


# ---------------------------------------------------------------------------
# bias-GeLU
# ---------------------------------------------------------------------------
def bias_gelu_fwd(x, bias, out="f64", acc=np.float64):
    """functional.py:37-40 (bias) / :23-25 (no bias), tanh approximation."""
    u = np.asarray(x, dtype=acc)
    if bias is not None:
        u = u + np.asarray(bias, dtype=acc)
    y = u * 0.5 * (1.0 + np.tanh(GELU_A * u * (1 + GELU_B * u * u)))
    return round_to(y, out)


def bias_gelu_bwd(g, x, bias, out="f64", acc=np.float64):
    """Returns (dx, dbias).  functional.py:43-50; dbias is the column sum of dx
    AS STORED (autograd sum-reduces the rounded full-size tensor that
    functional.py:84 returns for the bias)."""
    u = np.asarray(x, dtype=acc)
    if bias is not None:
        u = u + np.asarray(bias, dtype=acc)
    t = np.tanh(GELU_A * u * (1 + GELU_B * u * u))
    ff = 0.5 * u * ((1 - t * t) * (GELU_A + GELU_C * u * u)) + 0.5 * (1 + t)
    dx = round_to(ff * np.asarray(g, dtype=acc), out)
    if bias is None:
        return dx, None
    cols = dx.shape[-1]
    dbias = np.asarray(dx, dtype=acc).reshape(-1, cols).sum(axis=0)
    return dx, round_to(dbias, out)


# ---------------------------------------------------------------------------
# bias-dropout-add
# ---------------------------------------------------------------------------
def bias_dropout_add_fwd(x, bias, residual, keep, p, out="f64", acc=np.float64):
    """out = keep * (x + bias) / (1 - p) + residual, rounded once.

    functional.py:295-298 (F.dropout(x + bias, p, training)) followed by the
    caller's residual add (modeling_gpt2.py:369, 396).  `keep` is the 0/1 mask
    (None = keep everything, i.e. p == 0 or eval mode).
    """
    t = np.asarray(x, dtype=acc)
    if bias is not None:
        t = t + np.asarray(bias, dtype=acc)
    if keep is not None:
        scale = acc(np.float32(1.0) / (np.float32(1.0) - np.float32(p))) if p < 1.0 else acc(0.0)
        t = np.where(np.asarray(keep, dtype=bool), t * scale, 0.0)
    if residual is not None:
        t = t + np.asarray(residual, dtype=acc)
    return round_to(t, out)


def bias_dropout_add_bwd(g, keep, p, out="f64", acc=np.float64):
    """Returns (dx, dbias): dx = keep * g / (1 - p); dbias = column sum of dx as
    stored; the residual's gradient is g itself."""
    t = np.asarray(g, dtype=acc)
    if keep is not None:
        scale = acc(np.float32(1.0) / (np.float32(1.0) - np.float32(p))) if p < 1.0 else acc(0.0)
        t = np.where(np.asarray(keep, dtype=bool), t * scale, 0.0)
    dx = round_to(t, out)
    cols = dx.shape[-1]
    dbias = np.asarray(dx, dtype=acc).reshape(-1, cols).sum(axis=0)
    return dx, round_to(dbias, out)


# ---------------------------------------------------------------------------
# bias-dropout-add fused into the following norm
# ---------------------------------------------------------------------------
def bias_dropout_add_norm_fwd(x, bias, residual, keep, p, gamma, beta, eps, rms=False,
                              out="f64", acc=np.float64):
    """Returns (y, h, mean, invvar): h = dropout(x + bias) + residual rounded once
    to the storage type, y = LayerNorm / RMSNorm of that stored h.

    The chain FusedBiasDropout -> residual add -> LayerNorm of
    oslo/transformers/models/bert/modeling_bert.py:343-346; composed from
    bias_dropout_add_fwd and layer_norm_fwd / rms_norm_fwd above.  mean is None
    for RMSNorm.
    """
    h = bias_dropout_add_fwd(x, bias, residual, keep, p, out, acc)
    h = np.asarray(h, dtype=acc)
    if rms:
        y, invvar = rms_norm_fwd(h, gamma, eps, out, acc)
        return y, h, None, invvar
    y, mean, invvar = layer_norm_fwd(h, gamma, beta, eps, out, acc)
    return y, h, mean, invvar


def bias_dropout_add_norm_bwd(dy, dh_extra, h, mean, invvar, gamma, keep, p, rms=False,
                              out="f64", acc=np.float64):
    """Returns (dres, dx, dgamma, dbeta, dbias) of the fused chain.

    dh = norm_backward(dy) + dh_extra is formed in `acc`; dres = dh and
    dx = keep * dh / (1 - p) are each rounded once from it; dbias is the column
    sum of dx as stored; dgamma / dbeta as the plain norm backward (dbeta None
    for RMSNorm).
    """
    if rms:
        dh, dgamma = rms_norm_bwd(dy, h, invvar, gamma, "f64", out, acc)
        dbeta = None
    else:
        dh, dgamma, dbeta = layer_norm_bwd(dy, h, mean, invvar, gamma, "f64", out, acc)
    dh = np.asarray(dh, dtype=acc)
    if dh_extra is not None:
        dh = dh + np.asarray(dh_extra, dtype=acc)
    dres = round_to(dh, out)
    t = dh
    if keep is not None:
        t = np.where(np.asarray(keep, dtype=bool), dh * _dropout_scale(p, acc), 0.0)
    dx = round_to(t, out)
    n2 = dx.shape[-1]
    dbias = round_to(np.asarray(dx, dtype=acc).reshape(-1, n2).sum(axis=0), out)
    return dres, dx, dgamma, dbeta, dbias


# ---------------------------------------------------------------------------
# Adam / AdamW step
# ---------------------------------------------------------------------------
def adam_step(g, p, m, v, lr, beta1, beta2, eps, step, mode, bias_correction, weight_decay,
              out="f64", acc=np.float64):
    """One Adam update of one tensor; returns the new (p, m, v), each rounded
    once to the storage type.

    oslo/torch/_C/csrc/multi_tensor_adam.cu:78-96: mode 0 adds decay * p to the
    gradient (L2), mode 1 adds decay * p to the update (AdamW); the bias
    corrections 1 - beta^step are formed from the float32 betas and stored as
    float32 (:120-125); lr, eps, decay and the betas enter as float32 values.
    """
    f = lambda x: acc(np.float32(x))
    b1, b2 = f(beta1), f(beta2)
    bc1 = bc2 = acc(1.0)
    if bias_correction:
        bc1 = acc(np.float32(1.0 - float(np.float32(beta1)) ** step))
        bc2 = acc(np.float32(1.0 - float(np.float32(beta2)) ** step))
    g = np.asarray(g, dtype=acc)
    p = np.asarray(p, dtype=acc)
    m = np.asarray(m, dtype=acc)
    v = np.asarray(v, dtype=acc)
    if mode == 0:
        g = g + f(weight_decay) * p
    m = b1 * m + (acc(1.0) - b1) * g
    v = b2 * v + (acc(1.0) - b2) * g * g
    update = (m / bc1) / (np.sqrt(v / bc2) + f(eps))
    if mode != 0:
        update = update + f(weight_decay) * p
    p = p - f(lr) * update
    return round_to(p, out), round_to(m, out), round_to(v, out)


# ---------------------------------------------------------------------------
# SGD, Adagrad, NovoGrad, LAMB steps and the tensor norms they use
# ---------------------------------------------------------------------------
def _f32(x, acc):
    """A scalar argument as the kernel receives it: a float32 value."""
    return acc(np.float32(x))


def sgd_step(g, w, mom, lr, weight_decay, momentum, dampening, nesterov, first_run,
             wd_after_momentum=False, scale=1.0, out="f64", copy=None, acc=np.float64):
    """One SGD update of one tensor; returns the new ``(w, mom, w_copy)``.

    oslo/torch/_C/csrc/multi_tensor_sgd.cu:87-117: the gradient is multiplied
    by ``scale``; weight decay joins it before (default) or after the momentum
    step; on the first run the momentum buffer becomes the gradient, afterwards
    ``momentum * mom + (1 - dampening) * g``; Nesterov adds ``momentum * mom``
    to the gradient, plain momentum replaces the gradient by the buffer; the
    weight moves by ``-lr * g`` and is rounded to its storage type; ``w_copy``
    is that stored weight converted to the 16-bit type ``copy`` (:112-113).
    ``mom`` is returned unchanged when ``momentum == 0`` (never written, :116)."""
    g = np.asarray(g, dtype=acc) * _f32(scale, acc)
    w = np.asarray(w, dtype=acc)
    mom = np.asarray(mom, dtype=acc)
    wd, mu = _f32(weight_decay, acc), _f32(momentum, acc)
    if weight_decay != 0 and not wd_after_momentum:
        g = g + wd * w
    new_mom = mom
    if momentum != 0:
        # 1 - dampening is formed in float32 (:97), which is not exact for 0.1
        keep = acc(np.float32(1.0) - np.float32(dampening))
        new_mom = g if first_run else mom * mu + keep * g
        g = g + mu * new_mom if nesterov else new_mom
    if weight_decay != 0 and wd_after_momentum:
        g = g + wd * w
    w_new = round_to(w + (-_f32(lr, acc) * g), out)
    w_copy = None if copy is None else round_to(w_new, copy)
    return w_new, (round_to(new_mom, out) if momentum != 0 else mom), w_copy


def adagrad_step(g, p, h, lr, eps, mode, weight_decay, out="f64", acc=np.float64):
    """One Adagrad update; returns the new ``(p, h)``.

    oslo/torch/_C/csrc/multi_tensor_adagrad.cu:63-73: mode 0 adds ``decay * p``
    to the gradient (L2), mode 1 adds ``decay * p`` to the step; ``h`` is the
    running sum of squared gradients."""
    g = np.asarray(g, dtype=acc)
    p = np.asarray(p, dtype=acc)
    h = np.asarray(h, dtype=acc)
    lr_, eps_, wd = _f32(lr, acc), _f32(eps, acc), _f32(weight_decay, acc)
    if mode == 0:
        g = g + wd * p
        h = h + g * g
        p = p - lr_ * (g / (np.sqrt(h) + eps_))
    else:
        h = h + g * g
        p = p - lr_ * (g / (np.sqrt(h) + eps_) + wd * p)
    return round_to(p, out), round_to(h, out)


def tensor_norm(x, norm_type=2, acc=np.float64):
    """L2 norm (``norm_type`` 2) or largest magnitude (0) of one tensor
    (oslo/torch/_C/csrc/multi_tensor_l2norm.cu:62-98, 135-172)."""
    x = np.asarray(x, dtype=acc).reshape(-1)
    if x.size == 0:
        return acc(0.0)
    return np.sqrt(np.sum(x * x)) if norm_type == 2 else np.max(np.abs(x))


def blend_norm(old, x, alpha, beta, norm_type=2, acc=np.float64):
    """The stored per-tensor norm after a step (multi_tensor_l2norm.cu:319-322,
    226-253): L2 ``sqrt(alpha * old**2 + beta * |x|_2**2)``, max
    ``alpha * old + beta * max|x|``."""
    a, b = _f32(alpha, acc), _f32(beta, acc)
    n = tensor_norm(x, norm_type, acc)
    if norm_type == 2:
        return np.sqrt(a * acc(old) * acc(old) + b * n * n)
    return a * acc(old) + b * n


def novograd_step(g, p, m, grad_norm, lr, beta1, beta2, eps, step, bias_correction,
                  weight_decay, grad_averaging, moment_mode, out="f64", acc=np.float64):
    """The element-wise part of one NovoGrad update; ``grad_norm`` is the
    tensor's blended gradient norm (``blend_norm``).  Returns the new ``(p, m)``.

    oslo/torch/_C/csrc/multi_tensor_novograd.cu:80-96 and host code :118-129:
    ``bc1 = 1 - beta1**step``, ``bc2 = sqrt(1 - beta2**step)`` (float32),
    ``beta3 = 1 - beta1`` with gradient averaging, else 1."""
    g = np.asarray(g, dtype=acc)
    p = np.asarray(p, dtype=acc)
    m = np.asarray(m, dtype=acc)
    b1 = _f32(beta1, acc)
    bc1 = bc2 = acc(1.0)
    if bias_correction:
        bc1 = acc(np.float32(1.0 - float(np.float32(beta1)) ** step))
        bc2 = acc(np.float32(np.sqrt(1.0 - float(np.float32(beta2)) ** step)))
    b3 = acc(1.0) - b1 if grad_averaging else acc(1.0)
    denom = acc(grad_norm) / bc2 + _f32(eps, acc)
    wd, lr_ = _f32(weight_decay, acc), _f32(lr, acc)
    if moment_mode == 0:
        g = g / denom + wd * p
        m = b1 * m + b3 * g
        p = p - lr_ * (m / bc1)
    else:
        m = b1 * m + b3 * g
        p = p - lr_ * ((m / bc1) / denom + wd * p)
    return round_to(p, out), round_to(m, out)


def lamb_stage1(g, p, m, v, beta1, beta2, eps, step, bias_correction, weight_decay,
                grad_averaging, mode, global_grad_norm, max_grad_norm, out="f64",
                acc=np.float64, inv_scale=1.0, out_update=None):
    """LAMB stage 1 for one tensor: returns ``(update, m, v)``
    (oslo/torch/_C/csrc/multi_tensor_lamb.cu:111-130; bias corrections and
    beta3 from the host code :300-311).  ``inv_scale`` multiplies the gradient
    first, as the mixed-precision variant does (multi_tensor_lamb_mp.cu:111),
    whose update has the gradients' storage type ``out_update`` while the
    moments have the parameters' (``out``)."""
    g = np.asarray(g, dtype=acc) * acc(np.float32(inv_scale))
    p = np.asarray(p, dtype=acc)
    m = np.asarray(m, dtype=acc)
    v = np.asarray(v, dtype=acc)
    b1, b2 = _f32(beta1, acc), _f32(beta2, acc)
    bc1 = bc2 = acc(1.0)
    if bias_correction:
        bc1 = acc(np.float32(1.0 - float(np.float32(beta1)) ** step))
        bc2 = acc(np.float32(1.0 - float(np.float32(beta2)) ** step))
    b3 = acc(1.0) - b1 if grad_averaging else acc(1.0)
    gn, mx = acc(global_grad_norm), _f32(max_grad_norm, acc)
    clip = gn / mx if gn > mx else acc(1.0)
    wd = _f32(weight_decay, acc)
    g = g / clip
    if mode == 0:
        g = g + wd * p
    m = m * b1 + b3 * g
    v = v * b2 + (acc(1.0) - b2) * g * g
    update = (m / bc1) / (np.sqrt(v / bc2) + _f32(eps, acc))
    if mode != 0:
        update = update + wd * p
    return round_to(update, out_update or out), round_to(m, out), round_to(v, out)


def lamb_stage2(update, p, param_norm, update_norm, lr, weight_decay, use_nvlamb, out="f64",
                acc=np.float64):
    """LAMB stage 2 for one tensor: ``p - ratio * update`` with the trust ratio
    ``lr * param_norm / update_norm`` for tensors under weight decay (every
    tensor with ``use_nvlamb``) when both norms are non-zero, else ``lr``
    (multi_tensor_lamb.cu:224-233, 262-264)."""
    ratio = _f32(lr, acc)
    if use_nvlamb or weight_decay != 0:
        if update_norm != 0 and param_norm != 0:
            ratio = _f32(lr, acc) * (acc(param_norm) / acc(update_norm))
    p = np.asarray(p, dtype=acc) - ratio * np.asarray(update, dtype=acc)
    return round_to(p, out)
