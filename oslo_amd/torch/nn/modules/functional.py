"""Autograd Functions and user functions of the fused non-GEMM ops.

Same names, argument order and defaults as the reference's
``oslo/torch/nn/modules/functional.py`` (Functions ``:53-230``, user functions
``:249-298``).  GPU tensors go to the HIP kernels through
``oslo_amd.torch._C``; CPU tensors take the same plain-torch formulas the
reference evaluates there (its TorchScript bodies ``:23-50, 295-298`` and the
module fallbacks ``layer_norm.py:17-30, 452-455``).
"""
import torch
from torch import Tensor  # noqa: F401  (named by the type comment of fused_bias_dropout)
from torch.nn import functional as F

from oslo_amd.torch._C import (
    get_fused_elementwise_kernel,
    get_layernorm_kernel,
    get_softmax_kernel,
)

"""
Autograd Functions
"""


def _cast_if_autocast_enabled(*args):
    # functional.py:16-20 of the reference, with the torch.amp spellings
    if not torch.is_autocast_enabled("cuda"):
        return args
    dtype = torch.get_autocast_dtype("cuda")

    def cast(a):
        if isinstance(a, torch.Tensor) and a.is_floating_point() and a.is_cuda:
            return a.to(dtype)
        return a

    return tuple(cast(a) for a in args)


def _apply_outside_autocast(function, *args):
    """``function.apply`` on operands cast to the autocast dtype with autocast
    switched off (functional.py:249-284 of the reference); without an active
    autocast region neither step does anything and both are skipped."""
    if not torch.is_autocast_enabled("cuda"):
        return function.apply(*args)
    args = _cast_if_autocast_enabled(*args)
    with torch.amp.autocast("cuda", enabled=False):
        return function.apply(*args)


def _gelu_fwd_torch(x):
    # functional.py:23-25
    return x * 0.5 * (1.0 + torch.tanh(0.79788456 * x * (1 + 0.044715 * x * x)))


def _gelu_bwd_torch(g, x):
    # functional.py:28-34
    tanh_out = torch.tanh(0.79788456 * x * (1 + 0.044715 * x * x))
    ff = 0.5 * x * (
        (1 - tanh_out * tanh_out) * (0.79788456 + 0.1070322243 * x * x)
    ) + 0.5 * (1 + tanh_out)
    return ff * g


class _FusedGeLUFunction(torch.autograd.Function):
    """
    Kernel fusion function: GeLU
    """

    @staticmethod
    def forward(ctx, input):
        ctx.input_tensor = input
        if not input.is_cuda:
            return _gelu_fwd_torch(input)
        return get_fused_elementwise_kernel().bias_gelu_forward(input.contiguous(), None)

    @staticmethod
    def backward(ctx, grad_output):
        input = ctx.input_tensor
        if not input.is_cuda:
            return _gelu_bwd_torch(grad_output, input)
        grad_input, _ = get_fused_elementwise_kernel().bias_gelu_backward(
            grad_output.contiguous(), input.contiguous(), None
        )
        return grad_input


class _FusedBiasGeLUFunction(torch.autograd.Function):
    """
    Kernel fusion function: Bias + GeLU
    """

    @staticmethod
    def forward(ctx, input, bias):
        ctx.save_for_backward(input, bias)
        if not input.is_cuda:
            return _gelu_fwd_torch(input + bias)
        return get_fused_elementwise_kernel().bias_gelu_forward(
            input.contiguous(), bias.contiguous()
        )

    @staticmethod
    def backward(ctx, grad_output):
        input, bias = ctx.saved_tensors
        if not input.is_cuda:
            # the reference returns the full-size tensor twice and lets autograd
            # sum it down to the bias shape (functional.py:80-84)
            tmp = _gelu_bwd_torch(grad_output, input + bias)
            return tmp, tmp
        grad_input, grad_bias = get_fused_elementwise_kernel().bias_gelu_backward(
            grad_output.contiguous(),
            input.contiguous(),
            bias.contiguous(),
            need_bias_grad=ctx.needs_input_grad[1],
        )
        return grad_input, grad_bias


class _FusedBiasDropoutAddFunction(torch.autograd.Function):
    """
    Kernel fusion function: Bias + Dropout (+ residual add)

    The keep mask is a pure function of (seed, offset, element index) and is
    regenerated in backward, never stored.
    """

    @staticmethod
    def forward(ctx, input, bias, residual, p, seed, offset, inplace):
        kernel = get_fused_elementwise_kernel()
        input_ = input.contiguous()
        with _rng(seed):
            out = kernel.bias_dropout_add_forward(
                input_,
                None if bias is None else bias.contiguous(),
                None if residual is None else residual.contiguous(),
                p,
                _seed_arg(seed),
                offset,
                out=input_ if (inplace and input_ is input) else None,
            )
        if inplace and input_ is input:
            ctx.mark_dirty(input)
        ctx.p, ctx.seed, ctx.offset = p, seed, offset
        ctx.has_bias = bias is not None
        ctx.has_residual = residual is not None
        return out

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        need_x = ctx.needs_input_grad[0]
        need_b = ctx.has_bias and ctx.needs_input_grad[1]
        need_r = ctx.has_residual and ctx.needs_input_grad[2]
        with _rng(ctx.seed):
            grad_input, grad_bias = get_fused_elementwise_kernel().bias_dropout_add_backward(
                grad_output, ctx.p, _seed_arg(ctx.seed), ctx.offset,
                need_input_grad=need_x, need_bias_grad=need_b,
            )
        return grad_input, grad_bias, (grad_output if need_r else None), None, None, None, None


# Dropout state in device memory, one per device, for launches captured in a
# graph: {seed, offset} as two int64.  Created by the first eager dropout call
# on the device (a host-to-device copy cannot be captured) and re-seeded in
# place when torch's seed changes; its offsets start 2^40 above the generator's
# so that the two sequences stay apart.
_graph_rng = {}


def _as_i64(v):
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >= (1 << 63) else v


def _graph_rng_state(index, seed, offset):
    """The state tensor of device `index`, created on first use and never
    replaced: captured graphs hold its address, so a new seed is written into
    the same memory (eager calls only; nothing is captured here)."""
    entry = _graph_rng.get(index)
    if entry is None:
        state = torch.tensor([_as_i64(seed), _as_i64(offset + (1 << 40))], dtype=torch.int64,
                             device=torch.device("cuda", index))
        _graph_rng[index] = [seed, state]
        return state
    if entry[0] != seed:
        entry[1].copy_(torch.tensor([_as_i64(seed), _as_i64(offset + (1 << 40))], dtype=torch.int64))
        entry[0] = seed
    return entry[1]


def _next_philox_state(device):
    """(seed, offset) for one dropout call.

    Eager: the pair comes from torch's generator of `device`, whose offset
    advances by 4.  During stream capture the host cannot read the generator
    (and a pair baked into the graph would repeat one mask on every replay):
    ``seed`` is then a snapshot of the device-resident state -- a tensor that
    the kernels read when they run -- and that state advances by a captured
    add, so every replay draws new masks.  Backward takes the same pair."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if torch.cuda.is_current_stream_capturing():
        entry = _graph_rng.get(index)
        if entry is None:
            raise RuntimeError(
                "dropout with p > 0 is being captured in a graph before any eager dropout "
                "call on this device: run one eager step first (it creates the dropout "
                "state in device memory that captured launches read)."
            )
        state = entry[1]
        snapshot = state.clone()
        state[1:2].add_(4)
        return snapshot, 0
    gen = torch.cuda.default_generators[index]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + 4)
    _graph_rng_state(index, seed, offset)
    return seed, offset


def _rng(seed):
    """Context for a kernel call: a tensor `seed` is the device-resident pair."""
    from oslo_amd.torch._C import device_rng

    return device_rng(seed if isinstance(seed, torch.Tensor) else None)


def _seed_arg(seed):
    return 0 if isinstance(seed, torch.Tensor) else seed


def _norm_forward(ctx, rms, mixed, input, weight, bias, normalized_shape, eps):
    """Shared forward of the six norm Functions: contiguous operands in, stats
    saved for backward (mean only for LayerNorm)."""
    kernel = get_layernorm_kernel()
    ctx.normalized_shape = normalized_shape
    ctx.eps = eps
    ctx.rms = rms
    ctx.affine = weight is not None
    x = input.contiguous()
    if not ctx.affine:
        fwd = kernel.rms_norm_forward if rms else kernel.layer_norm_forward
        output, *stats = fwd(x, normalized_shape, eps)
        ctx.save_for_backward(x, *stats)
        return output
    w = weight.contiguous()
    if rms:
        fwd = (
            kernel.rms_norm_forward_affine_mixed_dtypes
            if mixed
            else kernel.rms_norm_forward_affine
        )
        output, invvar = fwd(x, normalized_shape, w, eps)
        ctx.save_for_backward(x, w, invvar)
        return output
    b = bias.contiguous()
    fwd = (
        kernel.layer_norm_forward_affine_mixed_dtypes
        if mixed
        else kernel.layer_norm_forward_affine
    )
    output, mean, invvar = fwd(x, normalized_shape, w, b, eps)
    ctx.save_for_backward(x, w, b, mean, invvar)
    return output


def _norm_backward(ctx, grad_output):
    """Shared backward: returns (grad_input, grad_weight, grad_bias); the last
    two are None where the variant has no such parameter."""
    kernel = get_layernorm_kernel()
    g = grad_output.contiguous()
    shape, eps = ctx.normalized_shape, ctx.eps
    saved = ctx.saved_tensors
    if not ctx.affine:
        if ctx.rms:
            x, invvar = saved
            return kernel.rms_norm_backward(g, invvar, x, shape, eps), None, None
        x, mean, invvar = saved
        return kernel.layer_norm_backward(g, mean, invvar, x, shape, eps), None, None
    if ctx.rms:
        x, w, invvar = saved
        gi, gw = kernel.rms_norm_backward_affine(g, invvar, x, shape, w, eps)
        return gi, gw, None
    x, w, b, mean, invvar = saved
    gi, gw, gb = kernel.layer_norm_backward_affine(g, mean, invvar, x, shape, w, b, eps)
    return gi, gw, gb


class _FusedLayerNormAffineFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, bias, normalized_shape, eps):
        return _norm_forward(ctx, False, False, input, weight, bias, normalized_shape, eps)

    @staticmethod
    def backward(ctx, grad_output):
        gi, gw, gb = _norm_backward(ctx, grad_output)
        return gi, gw, gb, None, None


class _FusedRMSNormAffineFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, normalized_shape, eps):
        return _norm_forward(ctx, True, False, input, weight, None, normalized_shape, eps)

    @staticmethod
    def backward(ctx, grad_output):
        gi, gw, _ = _norm_backward(ctx, grad_output)
        return gi, gw, None, None


class _FusedLayerNormAffineMixedDtypesFunction(_FusedLayerNormAffineFunction):
    # output in the parameters' dtype; backward inherited
    @staticmethod
    def forward(ctx, input, weight, bias, normalized_shape, eps):
        return _norm_forward(ctx, False, True, input, weight, bias, normalized_shape, eps)


class _FusedRMSNormAffineMixedDtypesFunction(_FusedRMSNormAffineFunction):
    @staticmethod
    def forward(ctx, input, weight, normalized_shape, eps):
        return _norm_forward(ctx, True, True, input, weight, None, normalized_shape, eps)


class _FusedLayerNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, normalized_shape, eps):
        return _norm_forward(ctx, False, False, input, None, None, normalized_shape, eps)

    @staticmethod
    def backward(ctx, grad_output):
        return _norm_backward(ctx, grad_output)[0], None, None


class _FusedRMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, normalized_shape, eps):
        return _norm_forward(ctx, True, False, input, None, None, normalized_shape, eps)

    @staticmethod
    def backward(ctx, grad_output):
        return _norm_backward(ctx, grad_output)[0], None, None


class _FusedBiasDropoutAddNormFunction(torch.autograd.Function):
    """
    Kernel fusion function: Bias + Dropout + residual add + LayerNorm / RMSNorm

    ``h = dropout(input + bias) + residual; y = norm(h) * weight + norm_bias`` --
    the chain of oslo/transformers/models/bert/modeling_bert.py:343-346 in one
    pass.  Returns ``(y, h)``; a gradient arriving at ``h`` (a pre-LN block
    keeps it as the next residual) is added to the norm's input gradient inside
    the backward kernel.
    """

    @staticmethod
    def forward(ctx, input, bias, residual, weight, norm_bias, normalized_shape, eps,
                p, seed, offset, rms):
        kernel = get_layernorm_kernel()
        # an output nobody consumes (h of a post-LN block) gets no zero-filled
        # gradient: backward sees None and the kernel skips that operand
        ctx.set_materialize_grads(False)
        with _rng(seed):
            y, h, mean, invvar = kernel.bias_dropout_add_norm_forward(
                rms,
                input.contiguous(),
                None if bias is None else bias.contiguous(),
                None if residual is None else residual.contiguous(),
                normalized_shape,
                None if weight is None else weight.contiguous(),
                None if norm_bias is None else norm_bias.contiguous(),
                eps, p, _seed_arg(seed), offset,
            )
        ctx.rms, ctx.p, ctx.seed, ctx.offset = rms, p, seed, offset
        ctx.normalized_shape = normalized_shape
        ctx.has = (bias is not None, residual is not None, weight is not None,
                   norm_bias is not None)
        saved = [h, invvar]
        if not rms:
            saved.append(mean)
        if weight is not None:
            saved.append(weight)
        ctx.save_for_backward(*saved)
        return y, h

    @staticmethod
    def backward(ctx, grad_y, grad_h):
        saved = list(ctx.saved_tensors)
        h, invvar = saved[0], saved[1]
        mean = None if ctx.rms else saved[2]
        has_bias, has_res, has_weight, has_nbias = ctx.has
        weight = saved[-1] if has_weight else None
        need_b = has_bias and ctx.needs_input_grad[1]
        if grad_y is None:
            if grad_h is None:
                return (None,) * 11
            # only h was used: the backward of dropout(input + bias) + residual
            with _rng(ctx.seed):
                g_in, g_bias = get_fused_elementwise_kernel().bias_dropout_add_backward(
                    grad_h.contiguous(), ctx.p, _seed_arg(ctx.seed), ctx.offset,
                    need_input_grad=ctx.needs_input_grad[0], need_bias_grad=need_b,
                )
            return (g_in, g_bias if need_b else None, grad_h if has_res else None,
                    None, None, None, None, None, None, None, None)
        if _fused_norm_backward_spills(h, ctx.normalized_shape):
            return _FusedBiasDropoutAddNormFunction._composed_backward(
                ctx, grad_y, grad_h, h, mean, invvar, weight, need_b)
        with _rng(ctx.seed):
            g_res, g_in, g_gamma, g_beta, g_bias = (
                get_layernorm_kernel().bias_dropout_add_norm_backward(
                    ctx.rms, grad_y.contiguous(),
                    None if grad_h is None else grad_h.contiguous(),
                    h, mean, invvar, ctx.normalized_shape, weight,
                    ctx.p, _seed_arg(ctx.seed), ctx.offset, need_bias_grad=need_b,
                )
            )
        return (
            g_in,
            g_bias if need_b else None,
            g_res if has_res else None,
            g_gamma if has_weight else None,
            g_beta if has_nbias else None,
            None, None, None, None, None, None,
        )


def _fused_norm_backward_spills(h, normalized_shape):
    """Rows for which the one-kernel backward of bias-dropout-add + norm holds
    more per lane than its 1024-lane workgroup has registers for (three column
    accumulators next to two operands): beyond 12288 16-bit or 6144 float32
    elements it spills and runs at a fraction of its rate (measured at
    [4096, 16384] bf16: 299 us against 141 us for the two backward kernels it
    fuses)."""
    n2 = 1
    for d in normalized_shape:
        n2 *= int(d)
    return n2 > (12288 if h.element_size() == 2 else 6144)


def _composed_fused_norm_backward(ctx, grad_y, grad_h, h, mean, invvar, weight, need_b):
    """The same gradients from the norm's backward kernel followed by the
    bias-dropout-add backward kernel (what the unfused modules run): the
    gradient of h is rounded to its dtype between the two."""
    kernel = get_layernorm_kernel()
    has_bias, has_res, has_weight, has_nbias = ctx.has
    grad_y = grad_y.contiguous()
    g_gamma = g_beta = None
    if ctx.rms:
        if has_weight:
            dh, g_gamma = kernel.rms_norm_backward_affine(
                grad_y, invvar, h, ctx.normalized_shape, weight, 0.0)
        else:
            dh = kernel.rms_norm_backward(grad_y, invvar, h, ctx.normalized_shape, 0.0)
    elif has_weight:
        dh, g_gamma, g_beta = kernel.layer_norm_backward_affine(
            grad_y, mean, invvar, h, ctx.normalized_shape, weight, weight, 0.0)
    else:
        dh = kernel.layer_norm_backward(grad_y, mean, invvar, h, ctx.normalized_shape, 0.0)
    if grad_h is not None:
        dh += grad_h
    with _rng(ctx.seed):
        g_in, g_bias = get_fused_elementwise_kernel().bias_dropout_add_backward(
            dh, ctx.p, _seed_arg(ctx.seed), ctx.offset,
            need_input_grad=ctx.needs_input_grad[0] and ctx.p > 0.0, need_bias_grad=need_b,
        )
    if ctx.p == 0.0:
        g_in = dh
    if g_bias is not None:
        g_bias = g_bias.view(tuple(int(d) for d in ctx.normalized_shape))
    return (
        g_in if ctx.needs_input_grad[0] else None,
        g_bias if need_b else None,
        dh if has_res else None,
        g_gamma if has_weight else None,
        g_beta if has_nbias else None,
        None, None, None, None, None, None,
    )


_FusedBiasDropoutAddNormFunction._composed_backward = staticmethod(_composed_fused_norm_backward)


class _ScaledUpperTriangMaskedSoftmax(torch.autograd.Function):
    """
    Fused: scale -> causal (upper-triangular) mask -> softmax, on
    [attn_batches, sq, sk] (FusedScaleMaskSoftmaxBinder.cpp:76-105).
    Saves the output only; backward is scale * y * (g - sum(g * y)).
    """

    @staticmethod
    def forward(ctx, inputs, scale):
        scale = float(scale)
        softmax_results = (
            get_softmax_kernel().fused_scaled_upper_triang_masked_softmax_forward(
                inputs.contiguous(), scale
            )
        )
        ctx.scale = scale
        ctx.save_for_backward(softmax_results)
        return softmax_results

    @staticmethod
    def backward(ctx, output_grads):
        (softmax_results,) = ctx.saved_tensors
        input_grads = (
            get_softmax_kernel().fused_scaled_upper_triang_masked_softmax_backward(
                output_grads.contiguous(), softmax_results, ctx.scale
            )
        )
        return input_grads, None


class _ScaledMaskedSoftmax(torch.autograd.Function):
    """
    Fused: scale -> padding mask -> softmax, on [b, np, sq, sk] with a
    [b or 1, 1, sq or 1, sk] mask, True = masked out
    (FusedScaleMaskSoftmaxBinder.cpp:39-70).  ``causal=True`` hides the keys
    beyond the diagonal as well, the combination a causal model applies to a
    padded batch (oslo/transformers/models/gpt2/modeling_gpt2.py:126-136).
    """

    @staticmethod
    def forward(ctx, inputs, mask, scale, causal=False):
        scale = float(scale)
        softmax_results = get_softmax_kernel().fused_scaled_masked_softmax_forward(
            inputs.contiguous(), mask, scale, causal=causal
        )
        ctx.scale, ctx.causal = scale, bool(causal)
        ctx.save_for_backward(softmax_results, mask)
        return softmax_results

    @staticmethod
    def backward(ctx, output_grads):
        softmax_results, mask = ctx.saved_tensors
        input_grads = get_softmax_kernel().fused_scaled_masked_softmax_backward(
            output_grads.contiguous(), softmax_results, ctx.scale, mask=mask, causal=ctx.causal
        )
        return input_grads, None, None, None


class _ScaledMaskedSoftmaxDropout(torch.autograd.Function):
    """
    Fused: scale -> causal or padding mask -> softmax -> dropout, the pair
    ``nn.functional.softmax`` + ``attn_dropout`` of
    oslo/transformers/models/gpt2/modeling_gpt2.py:138-142 and
    oslo/transformers/models/bert/modeling_bert.py:306-310 in one pass.

    ``mask=None``: causal, inputs [attn_batches, sq, sk]; otherwise inputs
    [b, np, sq, sk] with a padding mask.  Saves the *input* and two floats per
    row; backward recomputes the probabilities and regenerates the keep bits
    from (seed, offset), so neither the probabilities nor a mask are stored.
    """

    @staticmethod
    def forward(ctx, inputs, mask, scale, p, seed, offset, causal=False):
        scale = float(scale)
        inputs = inputs.contiguous()
        with _rng(seed):
            out, stats = get_softmax_kernel().softmax_dropout_forward(
                inputs, mask, scale, p, _seed_arg(seed), offset, causal=causal
            )
        ctx.scale, ctx.p, ctx.seed, ctx.offset = scale, p, seed, offset
        ctx.causal = bool(causal)
        ctx.has_mask = mask is not None
        if mask is not None:
            ctx.save_for_backward(inputs, stats, mask)
        else:
            ctx.save_for_backward(inputs, stats)
        return out

    @staticmethod
    def backward(ctx, output_grads):
        if ctx.has_mask:
            inputs, stats, mask = ctx.saved_tensors
        else:
            (inputs, stats), mask = ctx.saved_tensors, None
        with _rng(ctx.seed):
            input_grads = get_softmax_kernel().softmax_dropout_backward(
                output_grads.contiguous(), inputs, stats, mask, ctx.scale, ctx.p,
                _seed_arg(ctx.seed), ctx.offset, causal=ctx.causal,
            )
        return input_grads, None, None, None, None, None, None


def _bias_grad(dt, bias):
    """Gradient of an additive term from the gradient of the sum it was
    added into: summed over the dimensions the term was broadcast along, as
    autograd does for ``scores + term``."""
    g = dt.sum_to_size(bias.shape) if tuple(dt.shape) != tuple(bias.shape) else dt
    return g.to(bias.dtype)


class _ScaledBiasSoftmax(torch.autograd.Function):
    """
    Fused: ``softmax(scale * inputs + bias)`` on [b, np, sq, sk], the scores
    with an additive mask or bias
    (oslo/transformers/models/bert/modeling_bert.py:298-306,
    oslo/transformers/models/t5/modeling_t5.py:508-514); ``causal=True`` hides
    the keys beyond the diagonal as well.  Saves the output; the gradient of
    the term, when it is asked for, is the gradient of the sum reduced over the
    broadcast dimensions.
    """

    @staticmethod
    def forward(ctx, inputs, bias, scale, causal=False):
        scale = float(scale)
        softmax_results = get_softmax_kernel().softmax_bias_forward(
            inputs.contiguous(), bias, scale, causal=causal
        )
        ctx.scale, ctx.causal = scale, bool(causal)
        ctx.save_for_backward(softmax_results, bias)
        return softmax_results

    @staticmethod
    def backward(ctx, output_grads):
        softmax_results, bias = ctx.saved_tensors
        kernel = get_softmax_kernel()
        g = output_grads.contiguous()
        if not ctx.needs_input_grad[1]:
            dx = kernel.softmax_bias_backward(g, softmax_results, ctx.scale, bias=bias,
                                              causal=ctx.causal)
            return dx, None, None, None
        # gradient of the sum first (scale 1), then the two operands' shares
        dt = kernel.softmax_bias_backward(g, softmax_results, 1.0, bias=bias, causal=ctx.causal)
        dx = None
        if ctx.needs_input_grad[0]:
            dx = dt if ctx.scale == 1.0 else dt * ctx.scale
        return dx, _bias_grad(dt, bias), None, None


class _ScaledBiasSoftmaxDropout(torch.autograd.Function):
    """
    Fused: ``dropout(softmax(scale * inputs + bias), p)``; saves the inputs
    and two floats per row (see ``_ScaledMaskedSoftmaxDropout``).
    """

    @staticmethod
    def forward(ctx, inputs, bias, scale, p, seed, offset, causal=False):
        scale = float(scale)
        inputs = inputs.contiguous()
        with _rng(seed):
            out, stats = get_softmax_kernel().softmax_bias_dropout_forward(
                inputs, bias, scale, p, _seed_arg(seed), offset, causal=causal
            )
        ctx.scale, ctx.p, ctx.seed, ctx.offset = scale, p, seed, offset
        ctx.causal = bool(causal)
        ctx.save_for_backward(inputs, stats, bias)
        return out

    @staticmethod
    def backward(ctx, output_grads):
        inputs, stats, bias = ctx.saved_tensors
        want_bias = ctx.needs_input_grad[1]
        with _rng(ctx.seed):
            dt = get_softmax_kernel().softmax_bias_dropout_backward(
                output_grads.contiguous(), inputs, bias, stats, ctx.scale, ctx.p,
                _seed_arg(ctx.seed), ctx.offset, causal=ctx.causal,
            )
        if not want_bias:
            return dt, None, None, None, None, None, None
        # (the kernel returns scale * d(sum): the term's share is that without the scale)
        db = _bias_grad(dt if ctx.scale == 1.0 else dt / ctx.scale, bias)
        return (dt if ctx.needs_input_grad[0] else None), db, None, None, None, None, None


"""
User Functions
"""


def fused_layer_norm_affine(input, weight, bias, normalized_shape, eps=1e-6):
    return _apply_outside_autocast(_FusedLayerNormAffineFunction, input, weight, bias, normalized_shape, eps)


def fused_layer_norm(input, normalized_shape, eps=1e-6):
    return _apply_outside_autocast(_FusedLayerNormFunction, input, normalized_shape, eps)


def mixed_dtype_fused_layer_norm_affine(
    input, weight, bias, normalized_shape, eps=1e-6
):
    return _apply_outside_autocast(_FusedLayerNormAffineMixedDtypesFunction, input, weight, bias, normalized_shape, eps)


def fused_rms_norm_affine(input, weight, normalized_shape, eps=1e-6):
    return _apply_outside_autocast(_FusedRMSNormAffineFunction, input, weight, normalized_shape, eps)


def fused_rms_norm(input, normalized_shape, eps=1e-6):
    return _apply_outside_autocast(_FusedRMSNormFunction, input, normalized_shape, eps)


def mixed_dtype_fused_rms_norm_affine(input, weight, normalized_shape, eps=1e-6):
    return _apply_outside_autocast(_FusedRMSNormAffineMixedDtypesFunction, input, weight, normalized_shape, eps)


_KERNEL_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def _elementwise_operands(x, bias, residual=None):
    """Operands of the element-wise kernels, which take one dtype and a bias
    of shape ``[x.shape[-1]]``.  The reference evaluates ``x + bias`` with
    torch's promotion and broadcasting (functional.py:36-50, 295-298), so it
    accepts whatever the model holds; here, inside an autocast region every
    floating-point operand is cast to the autocast dtype (what the norm
    wrappers do, functional.py:16-20 there), outside of one ``bias`` and
    ``residual`` follow ``x``.  Returns ``(x, bias, residual, fits)``; with
    ``fits`` False (a bias that is not such a vector, a residual of another
    shape, a dtype without a kernel) the caller evaluates the torch formula."""
    autocast = x.is_cuda and torch.is_autocast_enabled("cuda")
    if autocast:
        x, bias, residual = _cast_if_autocast_enabled(x, bias, residual)
    else:
        if bias is not None and bias.dtype != x.dtype:
            bias = bias.to(x.dtype)
        if residual is not None and residual.dtype != x.dtype:
            residual = residual.to(x.dtype)
    fits = (
        x.dim() >= 1
        and x.dtype in _KERNEL_DTYPES
        and (bias is None or (bias.dim() == 1 and bias.shape[0] == x.shape[-1] and bias.device == x.device))
        and (residual is None or (residual.shape == x.shape and residual.device == x.device))
    )
    return x, bias, residual, fits


def _outside_autocast(x):
    """Context in which a Function runs on operands that were cast already."""
    if x.is_cuda and torch.is_autocast_enabled("cuda"):
        return torch.amp.autocast("cuda", enabled=False)
    return _NullContext()


class _NullContext:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


def _check_dropout_p(p):
    if p < 0.0 or p > 1.0:
        raise ValueError(
            "dropout probability has to be between 0 and 1, but got {}".format(p)
        )


def fused_gelu(x):
    if not x.is_cuda:
        return _FusedGeLUFunction.apply(x)
    x, _, _, fits = _elementwise_operands(x, None)
    with _outside_autocast(x):
        if not fits:
            return _gelu_fwd_torch(x)
        return _FusedGeLUFunction.apply(x)


def fused_bias_gelu(x, bias):
    if not x.is_cuda:
        return _FusedBiasGeLUFunction.apply(x, bias)
    x, bias, _, fits = _elementwise_operands(x, bias)
    with _outside_autocast(x):
        if not fits:
            return _gelu_fwd_torch(x + bias)
        return _FusedBiasGeLUFunction.apply(x, bias)


def fused_bias_dropout(x, bias, p, training, inplace):
    # type: (Tensor, Tensor, float, bool, bool) -> Tensor
    if not x.is_cuda:
        return F.dropout(x + bias, p=p, training=training, inplace=inplace)
    return fused_bias_dropout_add(x, bias, None, p, training, inplace)


def fused_bias_dropout_add(x, bias, residual, p, training, inplace=False):
    """dropout(x + bias) + residual in one kernel.

    The reference fuses only ``dropout(x + bias)`` (functional.py:295-298) and
    its callers add the residual next (modeling_gpt2.py:300, 369); passing the
    residual here folds that add into the same pass.  ``bias`` and ``residual``
    may be None.
    """
    _check_dropout_p(p)
    if not x.is_cuda:
        y = x if bias is None else x + bias
        y = F.dropout(y, p=p, training=training, inplace=inplace and bias is None)
        return y if residual is None else y + residual
    x_in = x
    x, bias, residual, fits = _elementwise_operands(x, bias, residual)
    with _outside_autocast(x):
        if not fits:
            y = x if bias is None else x + bias
            y = F.dropout(y, p=p, training=training)
            return y if residual is None else y + residual
        p_eff = float(p) if training else 0.0
        seed, offset = _next_philox_state(x.device) if p_eff > 0.0 else (0, 0)
        return _FusedBiasDropoutAddFunction.apply(
            x, bias, residual, p_eff, seed, offset, bool(inplace) and x is x_in
        )


def _bias_dropout_add_norm(rms, x, bias, residual, weight, norm_bias, normalized_shape,
                           eps, p, training, return_sum):
    _check_dropout_p(p)
    normalized_shape = (
        (int(normalized_shape),) if isinstance(normalized_shape, int)
        else tuple(int(s) for s in normalized_shape)
    )
    if not x.is_cuda:
        # the reference's CPU path: the unfused chain of torch ops
        h = x if bias is None else x + bias
        h = F.dropout(h, p=p, training=training)
        if residual is not None:
            h = h + residual
        if rms:
            from oslo_amd.torch.nn.modules.layer_norm import manual_rms_norm

            y = manual_rms_norm(h, normalized_shape, weight, eps)
        else:
            y = F.layer_norm(h, normalized_shape, weight, norm_bias, eps)
        return (y, h) if return_sum else y
    p_eff = float(p) if training else 0.0
    seed, offset = _next_philox_state(x.device) if p_eff > 0.0 else (0, 0)
    args = _cast_if_autocast_enabled(x, bias, residual, weight, norm_bias)
    with torch.amp.autocast("cuda", enabled=False):
        y, h = _FusedBiasDropoutAddNormFunction.apply(
            *args, normalized_shape, eps, p_eff, seed, offset, bool(rms)
        )
    return (y, h) if return_sum else y


def fused_bias_dropout_add_layer_norm(x, bias, residual, weight, norm_bias,
                                      normalized_shape, eps=1e-5, p=0.0, training=True,
                                      return_sum=False):
    """``LayerNorm(dropout(x + bias, p) + residual)`` in one kernel.

    The post-LN chain of oslo/transformers/models/bert/modeling_bert.py:343-346
    (FusedBiasDropout, residual add, nn.LayerNorm).  ``bias``, ``residual``,
    ``weight`` / ``norm_bias`` may be None.  With ``return_sum`` the normalised
    tensor comes with ``h = dropout(x + bias) + residual`` -- what a pre-LN block
    (modeling_gpt2.py:369-393) carries on as its residual.
    """
    return _bias_dropout_add_norm(False, x, bias, residual, weight, norm_bias,
                                  normalized_shape, eps, p, training, return_sum)


def fused_bias_dropout_add_rms_norm(x, bias, residual, weight, normalized_shape,
                                    eps=1e-5, p=0.0, training=True, return_sum=False):
    """``RMSNorm(dropout(x + bias, p) + residual)`` in one kernel (see above)."""
    return _bias_dropout_add_norm(True, x, bias, residual, weight, None,
                                  normalized_shape, eps, p, training, return_sum)


def scaled_upper_triang_masked_softmax(input, scale=1.0):
    """softmax(scale * input) under a causal mask; input is [attn_batches, sq, sk]."""
    return _ScaledUpperTriangMaskedSoftmax.apply(input, scale)


def scaled_masked_softmax(input, mask, scale=1.0, causal=False):
    """softmax(scale * input) with `mask` (True = masked out); input is [b, np, sq, sk].
    With ``causal=True`` key j of query i is hidden when j > i + (sk - sq) as well."""
    return _ScaledMaskedSoftmax.apply(input, mask, scale, causal)


def scaled_upper_triang_masked_softmax_dropout(input, scale=1.0, p=0.0, training=True):
    """dropout(softmax(scale * input) under a causal mask, p); [attn_batches, sq, sk]."""
    _check_dropout_p(p)
    p_eff = float(p) if training else 0.0
    if p_eff == 0.0:
        return _ScaledUpperTriangMaskedSoftmax.apply(input, scale)
    seed, offset = _next_philox_state(input.device)
    return _ScaledMaskedSoftmaxDropout.apply(input, None, scale, p_eff, seed, offset)


def scaled_masked_softmax_dropout(input, mask, scale=1.0, p=0.0, training=True, causal=False):
    """dropout(softmax(scale * input) with `mask`, p); input is [b, np, sq, sk];
    ``causal`` as in ``scaled_masked_softmax``."""
    _check_dropout_p(p)
    p_eff = float(p) if training else 0.0
    if p_eff == 0.0:
        return _ScaledMaskedSoftmax.apply(input, mask, scale, causal)
    seed, offset = _next_philox_state(input.device)
    return _ScaledMaskedSoftmaxDropout.apply(input, mask, scale, p_eff, seed, offset, causal)


def scaled_bias_softmax(input, bias, scale=1.0, causal=False):
    """softmax(scale * input + bias) over the last dimension; input is
    [b, np, sq, sk] and `bias` a floating-point tensor that broadcasts against
    it (an additive mask such as [b, 1, 1, sk] filled with -10000, the lowest
    finite value or -inf; a position bias [1, np, sq, sk]).  With
    ``causal=True`` key j of query i is hidden when j > i + (sk - sq) as well.
    `bias` may require a gradient."""
    return _ScaledBiasSoftmax.apply(input, bias, scale, causal)


def scaled_bias_softmax_dropout(input, bias, scale=1.0, p=0.0, training=True, causal=False):
    """dropout(softmax(scale * input + bias), p); see ``scaled_bias_softmax``."""
    _check_dropout_p(p)
    p_eff = float(p) if training else 0.0
    if p_eff == 0.0:
        return _ScaledBiasSoftmax.apply(input, bias, scale, causal)
    seed, offset = _next_philox_state(input.device)
    return _ScaledBiasSoftmaxDropout.apply(input, bias, scale, p_eff, seed, offset, causal)
