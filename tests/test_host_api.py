"""The Python layer without a GPU: the module / functional API mirrors the
reference's (names, constructor arguments, parameters, extra_repr, defaults) and
CPU tensors take the reference's own unfused torch path."""
import inspect
import warnings

import pytest
import torch

import oslo_amd.torch.nn as onn
from oracle import torch_path as tp
from oslo_amd.torch.nn.modules import functional as F_


def test_exports_match_reference_names():
    # oslo/torch/nn/__init__.py:1-53, the hot-path subset
    for name in [
        "FusedBiasDropout", "FusedLayerNorm", "FusedRMSNorm", "MixedFusedLayerNorm", "MixedFusedRMSNorm",
        "Conv1D", "Linear", "fused_bias_dropout", "fused_bias_gelu", "fused_gelu", "fused_rms_norm_affine",
        "fused_layer_norm", "mixed_dtype_fused_layer_norm_affine", "fused_layer_norm_affine",
        "mixed_dtype_fused_rms_norm_affine", "fused_rms_norm", "FusedScaleMaskSoftmax",
    ]:
        assert hasattr(onn, name), name


def test_functional_signatures_and_defaults():
    # functional.py:249-298 of the reference: eps defaults to 1e-6, positional order
    sig = inspect.signature(onn.fused_layer_norm_affine)
    assert list(sig.parameters) == ["input", "weight", "bias", "normalized_shape", "eps"]
    assert sig.parameters["eps"].default == 1e-6
    assert list(inspect.signature(onn.fused_rms_norm_affine).parameters) == ["input", "weight", "normalized_shape", "eps"]
    assert list(inspect.signature(onn.fused_layer_norm).parameters) == ["input", "normalized_shape", "eps"]
    assert list(inspect.signature(onn.fused_bias_dropout).parameters) == ["x", "bias", "p", "training", "inplace"]
    assert list(inspect.signature(onn.fused_bias_gelu).parameters) == ["x", "bias"]
    for fn in (onn.mixed_dtype_fused_layer_norm_affine, onn.mixed_dtype_fused_rms_norm_affine, onn.fused_rms_norm):
        assert inspect.signature(fn).parameters["eps"].default == 1e-6


@pytest.mark.parametrize("cls", [onn.FusedLayerNorm, onn.FusedRMSNorm])
def test_norm_module_construction(cls):
    m = cls(48)
    assert m.normalized_shape == torch.Size([48]) and m.eps == 1e-5 and m.elementwise_affine
    assert torch.equal(m.weight, torch.ones(48))
    if cls is onn.FusedLayerNorm:
        assert torch.equal(m.bias, torch.zeros(48))
        assert set(dict(m.named_parameters())) == {"weight", "bias"}
    else:
        assert set(dict(m.named_parameters())) == {"weight"}
    assert m.extra_repr() == "torch.Size([48]), eps=1e-05, elementwise_affine=True"
    m2 = cls([4, 6], eps=1e-3, elementwise_affine=False)
    assert m2.weight is None and m2.normalized_shape == torch.Size([4, 6])
    assert not isinstance(m, torch.nn.LayerNorm)  # tensor-parallel wrappers key on that
    sd = cls(8).state_dict()
    assert "weight" in sd


def test_norm_modules_cpu_path_is_the_reference_path():
    x = torch.randn(5, 7, 48)
    ln = onn.FusedLayerNorm(48)
    with torch.no_grad():
        ln.weight.uniform_(0.5, 1.5)
        ln.bias.uniform_(-0.5, 0.5)
    assert torch.equal(ln(x), tp.layer_norm(x, ln.weight, ln.bias, ln.eps))
    rms = onn.FusedRMSNorm(48)
    with torch.no_grad():
        rms.weight.uniform_(0.5, 1.5)
    assert torch.equal(rms(x), tp.rms_norm(x, rms.weight, rms.eps))
    # half-precision weights: the normalised value is cast to the weight dtype first
    rms16 = onn.FusedRMSNorm(48).to(torch.bfloat16)
    out = rms16(x.to(torch.bfloat16))
    assert out.dtype == torch.bfloat16
    assert torch.equal(out, tp.rms_norm(x.to(torch.bfloat16), rms16.weight, rms16.eps))
    # two trailing dimensions
    ln2 = onn.FusedLayerNorm([7, 48])
    assert torch.allclose(ln2(x), torch.nn.functional.layer_norm(x, (7, 48)))
    rms2 = onn.FusedRMSNorm([7, 48], elementwise_affine=False)
    want = x * torch.rsqrt(x.pow(2).mean((-1, -2), keepdim=True) + 1e-5)
    assert torch.allclose(rms2(x), want)


@pytest.mark.parametrize("cls", [onn.MixedFusedLayerNorm, onn.MixedFusedRMSNorm])
def test_mixed_modules_reject_non_affine(cls):
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        m = cls(16, elementwise_affine=True)
        assert any("does not support `elementwise_affine` argument" in str(x.message) for x in w)
    assert m.elementwise_affine
    with pytest.raises(RuntimeError, match="elementwise_affine = False"):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            cls(16, elementwise_affine=False)
    y = m(torch.randn(3, 16))
    assert y.shape == (3, 16)


def test_bias_gelu_cpu_forward_backward():
    x = torch.randn(6, 32, dtype=torch.float64, requires_grad=True)
    b = torch.randn(32, dtype=torch.float64, requires_grad=True)
    g = torch.randn(6, 32, dtype=torch.float64)
    y = onn.fused_bias_gelu(x, b)
    y.backward(g)
    xr, br = x.detach().clone().requires_grad_(), b.detach().clone().requires_grad_()
    yr = tp.bias_gelu(xr, br)
    yr.backward(g)
    assert torch.allclose(y, yr) and torch.allclose(x.grad, xr.grad, rtol=1e-7, atol=1e-9)
    assert b.grad.shape == (32,) and torch.allclose(b.grad, br.grad, rtol=1e-7, atol=1e-9)
    x2 = torch.randn(4, 8, dtype=torch.float64, requires_grad=True)
    onn.fused_gelu(x2).sum().backward()
    assert torch.allclose(x2.grad, tp.bias_gelu_grad(torch.ones(4, 8, dtype=torch.float64), x2.detach(), None))


def test_fused_bias_dropout_cpu():
    m = onn.FusedBiasDropout(p=0.3)
    assert isinstance(m, torch.nn.modules.dropout._DropoutNd) and m.p == 0.3 and not m.inplace
    x, b, r = torch.randn(64, 32), torch.randn(32), torch.randn(64, 32)
    m.eval()
    assert torch.equal(m(x, b), x + b)
    assert torch.equal(m(x, b, r), x + b + r)
    m.train()
    torch.manual_seed(0)
    y = m(x, b)
    torch.manual_seed(0)
    assert torch.equal(y, torch.nn.functional.dropout(x + b, 0.3, True))
    assert torch.equal(onn.fused_bias_dropout(x, b, 0.0, True, False), x + b)
    with pytest.raises(ValueError):
        onn.fused_bias_dropout_add(x, b, None, 1.5, True)


def test_softmax_module_cpu_and_flags():
    x = torch.randn(2, 3, 8, 8)
    causal = onn.FusedScaleMaskSoftmax(attn_mask_type=onn.AttnMaskType.causal, scale=0.5)
    y = causal(x, None)
    assert torch.allclose(y, tp.causal_softmax(x, 0.5), atol=1e-7)
    pad = torch.zeros(2, 8, dtype=torch.bool)
    pad[1, 5:] = True
    padding = onn.FusedScaleMaskSoftmax(attn_mask_type=onn.AttnMaskType.padding, scale=0.25)
    y = padding(x, pad.view(2, 1, 1, 8))
    assert torch.allclose(y, tp.padding_softmax(x, pad, 0.25), atol=1e-7)
    assert not padding.is_kernel_available(None, 2, 3, 8, 8, input=x)  # CPU tensor
    with pytest.raises(ValueError):
        onn.FusedScaleMaskSoftmax(input_in_fp16=True, input_in_bf16=True)
    with pytest.raises(ValueError):
        onn.FusedScaleMaskSoftmax(softmax_in_fp32=False, scale=2.0)
    with pytest.raises(RuntimeError):
        causal(x[0], None)
    filled = onn.attention_mask_func(torch.zeros(1, 1, 2, 2), torch.tensor([[[[False, True], [False, False]]]]))
    assert filled[0, 0, 0, 1] == -10000.0
    with pytest.raises(ValueError, match="between 0 and 1"):
        onn.FusedScaleMaskSoftmax(attn_dropout=1.5)
    # why a call would not reach the kernels, as the module reports it
    assert "does not broadcast" in padding._unfused_reason(torch.zeros(1, 1, 1, 1, 8, dtype=torch.bool), 2, 3, 8, 8)
    assert padding._unfused_reason(None, 0, 3, 8, 8) == "empty input"
    assert padding(torch.zeros(0, 3, 8, 8), None).shape == (0, 3, 8, 8)
    # the torch chain applies the module's own dropout: off in eval mode, in training mode zeros and 1 / (1 - p)
    drop = onn.FusedScaleMaskSoftmax(attn_mask_type=onn.AttnMaskType.causal, scale=0.5, attn_dropout=0.5)
    assert torch.equal(drop.eval()(x, None), y * 0 + causal(x, None))
    torch.manual_seed(0)
    yd = drop.train()(x, None)
    ref = causal(x, None)
    kept = yd != 0
    assert 0.2 < kept.float().mean().item() / (ref != 0).float().mean().item() < 0.8
    assert torch.allclose(yd[kept], 2.0 * ref[kept])


def test_operands_without_a_kernel_take_the_torch_formulas():
    """float64 has no element-wise kernel: the functions evaluate the reference's formulas with torch."""
    x = torch.randn(5, 16, dtype=torch.float64)
    b, r = torch.randn(16, dtype=torch.float64), torch.randn(5, 16, dtype=torch.float64)
    assert torch.allclose(onn.fused_gelu(x), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-7)
    assert torch.equal(onn.fused_bias_dropout_add(x, b, r, 0.0, True), x + b + r)
    assert torch.equal(onn.fused_bias_dropout_add(x, None, None, 0.5, False), x)
    # the CPU chain of the residual RMSNorm: the reference's manual_rms_norm (layer_norm.py:17-30) on the sum
    w = torch.rand(16) + 0.5
    xf, bf, rf = x.float(), b.float(), r.float()
    y, h = onn.fused_bias_dropout_add_rms_norm(xf, bf, rf, w, (16,), 1e-6, 0.0, False, True)
    assert torch.equal(h, xf + bf + rf)
    want = w * (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6))
    assert torch.allclose(y, want, atol=1e-6)


def test_residual_norm_module_without_parameters():
    m = onn.FusedBiasDropoutAddLayerNorm(16, p=0.0, elementwise_affine=False)
    assert m.weight is None and m.bias is None and "elementwise_affine=False" in repr(m)
    x, b, r = torch.randn(3, 16), torch.randn(16), torch.randn(3, 16)
    out = m(x, b, r)
    out = out[0] if isinstance(out, tuple) else out
    assert torch.allclose(out, torch.nn.functional.layer_norm(x + b + r, (16,), eps=m.eps), atol=1e-6)


def test_additive_term_operand_and_flags():
    """How the binding hands an additive term to the kernel: element strides of
    the batch / head / query dimensions (0 where the term broadcasts, expanded
    views included), float32 for a term in another type than the scores, and
    the default of the skip flag (backward passes of a term shared by heads or
    queries only).  Host logic: no GPU needed."""
    from oslo_amd.torch._C import _SoftmaxKernel as K

    x = torch.zeros(3, 4, 5, 8, dtype=torch.bfloat16)
    op = K._bias_operand
    t, sb, sh, sq, code = op(torch.zeros(3, 1, 1, 8, dtype=torch.bfloat16), x)
    assert (sb, sh, sq, code) == (8, 0, 0, 2) and t.shape == (3, 1, 1, 8)
    t, sb, sh, sq, code = op(torch.zeros(4, 5, 8, dtype=torch.bfloat16), x)      # [np, sq, sk]
    assert (sb, sh, sq) == (0, 40, 8) and t.dim() == 4
    base = torch.zeros(1, 4, 5, 8, dtype=torch.bfloat16)
    t, sb, sh, sq, code = op(base.expand(3, 4, 5, 8), x)                          # stride 0 kept
    assert (sb, sh, sq) == (0, 40, 8) and t.data_ptr() == base.data_ptr()
    t, sb, sh, sq, code = op(torch.zeros(8, dtype=torch.float16), x)              # another type -> float32
    assert (sb, sh, sq, code) == (0, 0, 0, 0) and t.dtype == torch.float32
    t, sb, sh, sq, code = op(torch.zeros(3, 4, 5, 8, dtype=torch.float64), x)
    assert t.dtype == torch.float32 and (sb, sh, sq) == (160, 40, 8)
    t, sb, sh, sq, code = op(torch.zeros(5, 1, dtype=torch.bfloat16), x)          # a column: expanded over the keys
    assert t.shape == (1, 1, 5, 8) and (sb, sh, sq) == (0, 0, 8) and t.stride(3) == 1
    wide = torch.zeros(5, 16, dtype=torch.bfloat16)
    t, sb, sh, sq, code = op(wide[:, ::2], x)                                     # keys not contiguous: copied
    assert t.stride(3) == 1 and sq == 8
    t, sb, sh, sq, code = op(wide[:, 3:11], x)                                    # rows 32 bytes apart stay a view
    assert sq == 16 and t.data_ptr() == wide.data_ptr() + 6
    for bad in (torch.zeros(2, 1, 1, 8), torch.zeros(3, 4, 5, 7), torch.zeros(1, 1, 1, 1, 8)):
        with pytest.raises(RuntimeError):
            op(bad, x)
    with pytest.raises(RuntimeError):
        op(torch.zeros(3, 1, 1, 8, dtype=torch.bool), x)
    with pytest.raises(RuntimeError):
        op(torch.zeros(8), x[0])
    fl = K._bias_flags
    assert fl(False, None, (8, 0, 0), True) == 0 and fl(True, None, (8, 0, 0), True) == 1
    assert fl(False, None, (8, 0, 0), False) == 2 and fl(True, None, (0, 40, 0), False) == 3
    assert fl(False, None, (160, 40, 8), False) == 0          # a dense term: reading it would cost a third stream
    assert fl(False, True, (160, 40, 8), True) == 2 and fl(True, False, (8, 0, 0), False) == 1


def test_skip_bias_add_producers():
    lin = onn.Linear(8, 12, skip_bias_add=True)
    out, bias = lin(torch.randn(3, 8))
    assert out.shape == (3, 12) and bias is lin.bias
    assert onn.Linear(8, 12)(torch.randn(3, 8)).shape == (3, 12)
    conv = onn.Conv1D(12, 8, skip_bias_add=True)
    assert conv.weight.shape == (8, 12) and conv.nf == 12
    out, bias = conv(torch.randn(2, 5, 8))
    assert out.shape == (2, 5, 12) and bias is conv.bias
    x = torch.randn(2, 5, 8)
    full = onn.Conv1D(12, 8)
    assert torch.allclose(full(x), x @ full.weight + full.bias, atol=1e-6)


def test_gpu_entry_points_refuse_cpu_tensors():
    from oslo_amd.torch import _C

    k = _C.get_layernorm_kernel()
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        k.layer_norm_forward(torch.zeros(2, 4), (4,), 1e-5)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        _C.get_softmax_kernel().fused_scaled_upper_triang_masked_softmax_forward(torch.zeros(1, 2, 2), 1.0)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        _C.get_fused_elementwise_kernel().bias_gelu_forward(torch.zeros(2, 8), None)
    # cast helper is the identity outside autocast
    a = torch.zeros(2)
    assert F_._cast_if_autocast_enabled(a, 3)[0] is a


def test_fused_optimizers_mirror_the_reference_constructors():
    """oslo/torch/optim/__init__.py:1-6: the class names, and the argument checks
    that need no GPU (fused_sgd.py:98-114, fused_novograd.py:86-87)."""
    import oslo_amd.torch.optim as optim

    for name in ("FusedAdam", "FusedAdagrad", "FusedLamb", "FusedMixedPrecisionLamb", "FusedNovograd",
                 "FusedSGD"):
        assert issubclass(getattr(optim, name), torch.optim.Optimizer)
    w = torch.nn.Parameter(torch.zeros(4))
    sgd = optim.FusedSGD([w], lr=0.1, momentum=0.9, nesterov=True)
    assert sgd.defaults == dict(lr=0.1, momentum=0.9, dampening=0, weight_decay=0, nesterov=True)
    assert sgd.wd_after_momentum is False and sgd.most_recent_scale == 1.0
    for bad in (dict(lr=-0.1), dict(lr=0.1, momentum=-1.0), dict(lr=0.1, weight_decay=-1.0),
                dict(lr=0.1, nesterov=True), dict(lr=0.1, momentum=0.9, dampening=0.1, nesterov=True)):
        with pytest.raises(ValueError):
            optim.FusedSGD([w], **bad)
    ada = optim.FusedAdagrad([w])
    assert ada.defaults == dict(lr=1e-3, eps=1e-10, weight_decay=0.0) and ada.adagrad_w_mode == 0
    novo = optim.FusedNovograd([w], reg_inside_moment=True)
    assert novo.moment_mode == 0 and novo.defaults["norm_type"] == 2 and novo.defaults["betas"] == (0.9, 0.999)
    with pytest.raises(RuntimeError):
        optim.FusedNovograd([w], amsgrad=True)
    lamb = optim.FusedLamb([w], max_grad_norm=1.0)
    assert lamb.defaults["max_grad_norm"] == 1.0 and lamb.adam_w_mode == 1
    with pytest.raises(RuntimeError):
        optim.FusedLamb([w], eps_inside_sqrt=True)
    # a step on CPU parameters is refused with a clear message, not attempted
    w.grad = torch.ones(4)
    with pytest.raises(RuntimeError, match="GPU-only"):
        sgd.step()
    # parameters without gradients: nothing to do, no GPU needed
    w.grad = None
    for opt in (sgd, ada, novo, lamb):
        opt.step()
