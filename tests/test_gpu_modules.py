"""The module / functional API on the GPU, in the design of the reference's own
tests (tests_deprecated/torch/_C/csrc/test_fused_layer_norm.py: the same module
built twice, once on the CPU = unfused torch path, once on the GPU = fused
kernels; outputs, input gradients and weight gradients compared), plus
autocast, strided inputs and the softmax / GeLU / dropout modules."""
import pytest
import torch

import oslo_amd.torch.nn as onn
from helpers import check, f64, randn

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16


def run_pair(cpu_mod, gpu_mod, x, dy, device, gpu_dtype=None):
    xc = x.clone().double().requires_grad_()
    cpu_mod = cpu_mod.double()
    yc = cpu_mod(xc)
    yc.backward(dy.double())
    xg = x.to(device)
    if gpu_dtype is not None:
        xg = xg.to(gpu_dtype)
    xg.requires_grad_()
    yg = gpu_mod(xg)
    yg.backward(dy.to(device).to(yg.dtype))
    return xc, yc, xg, yg


@pytest.mark.parametrize("cls", [onn.FusedLayerNorm, onn.FusedRMSNorm])
@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("contiguous", [True, False])
def test_norm_module_cpu_vs_gpu(device, cls, affine, dtype, contiguous):
    # normalized_shape=[32, 16] and batch 16 as in test_fused_layer_norm.py:104-108
    shape = [32, 16]
    torch.manual_seed(42)
    cpu = cls(shape, elementwise_affine=affine)
    gpu = cls(shape, elementwise_affine=affine)
    if affine:
        with torch.no_grad():
            # parameters representable in `dtype`, so both modules hold the
            # same values
            cpu.weight.copy_(randn(shape, dtype, 1, std=0.1, mean=1.0))
            if hasattr(cpu, "bias") and cpu.bias is not None:
                cpu.bias.copy_(randn(shape, dtype, 2, std=0.1))
        gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.to(device=device, dtype=dtype)
    if contiguous:
        x = randn([16] + shape, dtype, 3)
    else:
        # strided view as in test_fused_layer_norm.py:55-70
        x = randn([16, 32 * 3, 16 * 5], dtype, 3)[:, ::3, ::5]
        assert not x.is_contiguous()
    dy = randn([16] + shape, dtype, 4)
    xc, yc, xg, yg = run_pair(cpu, gpu, x, dy, device)
    assert yg.dtype == dtype and yg.shape == yc.shape
    rms16 = cls is onn.FusedRMSNorm and dtype != F32 and affine
    # RMS rounds the normalised value before the scale (two roundings), so a
    # float64 module is up to 2 ulp away; everything else rounds once
    check(yg, f64(yc), "module fwd", atol=2e-6, max_ulp=2 if rms16 else 1, min_exact=0.6 if rms16 else 0.998,
          l2_tol=4e-3 if rms16 else 2e-3)
    check(xg.grad, f64(xc.grad), "module dx", atol=4e-6)
    if affine:
        check(gpu.weight.grad, f64(cpu.weight.grad), "module dweight", atol=1e-4, min_exact=0.9)
        if getattr(gpu, "bias", None) is not None:
            check(gpu.bias.grad, f64(cpu.bias.grad), "module dbias", atol=1e-4, min_exact=0.9)


@pytest.mark.parametrize("cls", [onn.FusedLayerNorm, onn.FusedRMSNorm])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_norm_module_cpu_vs_gpu_large_batch(device, cls, dtype):
    """The reference's large case, tests_deprecated/torch/_C/csrc/
    test_fused_layer_norm.py:104-108: batch 65 536 of normalized_shape [32, 16]
    (33.5 M elements), the module on the CPU in float64 against the module on
    the GPU, forward and every gradient."""
    shape = [32, 16]
    batch = 65536
    torch.manual_seed(7)
    cpu = cls(shape)
    gpu = cls(shape)
    with torch.no_grad():
        cpu.weight.copy_(randn(shape, dtype, 1, std=0.1, mean=1.0))
        if getattr(cpu, "bias", None) is not None:
            cpu.bias.copy_(randn(shape, dtype, 2, std=0.1))
    gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.to(device=device, dtype=dtype)
    x = randn([batch] + shape, dtype, 3)
    dy = randn([batch] + shape, dtype, 4)
    xc, yc, xg, yg = run_pair(cpu, gpu, x, dy, device)
    rms16 = cls is onn.FusedRMSNorm and dtype != F32
    check(yg, f64(yc), "module fwd", atol=2e-6, max_ulp=2 if rms16 else 1, min_exact=0.6 if rms16 else 0.998,
          l2_tol=4e-3 if rms16 else 2e-3)
    check(xg.grad, f64(xc.grad), "module dx", atol=4e-6)
    # column sums over 65 536 rows: float32 accumulation of rounded terms against float64
    patol = 1e-5 * (batch ** 0.5) + 1e-4
    check(gpu.weight.grad, f64(cpu.weight.grad), "module dweight", atol=patol, min_exact=0.9)
    if getattr(gpu, "bias", None) is not None:
        check(gpu.bias.grad, f64(cpu.bias.grad), "module dbias", atol=patol, min_exact=0.9)


@pytest.mark.parametrize("cls", [onn.MixedFusedLayerNorm, onn.MixedFusedRMSNorm])
def test_mixed_modules_return_parameter_dtype(device, cls):
    m = cls(64).to(device=device, dtype=BF16)
    x = randn((8, 64), F32, 1).to(device).requires_grad_()
    y = m(x)
    assert y.dtype == BF16
    y.float().sum().backward()
    assert x.grad.dtype == F32 and m.weight.grad.dtype == BF16
    with pytest.warns(UserWarning):
        cls(64, elementwise_affine=True)
    with pytest.raises(RuntimeError):
        cls(64, elementwise_affine=False)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_norm_autocast_casts_inputs_and_output(device, dtype):
    # test_fused_layer_norm.py:296-321: under autocast the output has the
    # autocast dtype and matches torch.nn.LayerNorm run natively in that dtype
    m = onn.FusedLayerNorm(128).to(device)
    native = torch.nn.LayerNorm(128).to(device=device, dtype=dtype)
    x = randn((16, 128), F32, 5).to(device)
    with torch.autocast("cuda", dtype=dtype):
        y = m(x)
    assert y.dtype == dtype
    ref = native(x.to(dtype))
    assert (y == ref).double().mean() > 0.99
    assert (y.float() - ref.float()).abs().max() < 0.05


def test_functional_defaults_and_shapes(device):
    x = randn((4, 6, 48), F32, 1).to(device)
    w = torch.ones(48, device=device)
    b = torch.zeros(48, device=device)
    y = onn.fused_layer_norm_affine(x, w, b, (48,))  # eps defaults to 1e-6
    ref = torch.nn.functional.layer_norm(x.double(), (48,), None, None, 1e-6)
    check(y, f64(ref), "functional ln", atol=2e-6)
    y = onn.fused_rms_norm(x, (48,))
    ref = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-6)
    check(y, f64(ref), "functional rms", atol=2e-6)


def test_fused_bias_dropout_in_place(device):
    """inplace=True (functional.py:295-298 hands it to F.dropout): the result
    overwrites the input's memory, autograd is told so, and values and
    gradients equal those of the out-of-place call under the same seed."""
    x = randn((64, 256), BF16, 1).to(device).requires_grad_()
    b = randn((256,), BF16, 2, std=0.1).to(device).requires_grad_()
    g = randn((64, 256), BF16, 3).to(device)
    torch.manual_seed(7)
    ref = onn.fused_bias_dropout(x * 1, b, 0.25, True, False)
    ref.backward(g)
    gx, gb = x.grad.clone(), b.grad.clone()
    x.grad = b.grad = None
    h = x * 1
    torch.manual_seed(7)
    out = onn.fused_bias_dropout(h, b, 0.25, True, True)
    assert out.data_ptr() == h.data_ptr() and torch.equal(out, ref)
    out.backward(g)
    assert torch.equal(x.grad, gx) and torch.equal(b.grad, gb)
    with pytest.raises(RuntimeError):   # a leaf that requires a gradient cannot be overwritten
        onn.fused_bias_dropout(x, b, 0.25, True, True)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_fused_bias_gelu_autograd(device, dtype):
    x = randn((64, 256), dtype, 1)
    b = randn((256,), dtype, 2, std=0.1)
    g = randn((64, 256), dtype, 3)
    xd, bd = x.to(device).requires_grad_(), b.to(device).requires_grad_()
    y = onn.fused_bias_gelu(xd, bd)
    y.backward(g.to(device))
    xr, br = x.double().requires_grad_(), b.double().requires_grad_()
    yr = torch.nn.functional.gelu(xr + br, approximate="tanh")
    yr.backward(g.double())
    check(y, f64(yr), "fused_bias_gelu fwd", atol=1e-6)
    check(xd.grad, f64(xr.grad), "fused_bias_gelu dx", atol=2e-6)
    assert bd.grad.shape == (256,)
    check(bd.grad, f64(xd.grad).sum(0), "fused_bias_gelu dbias", atol=1e-4, min_exact=0.9)
    # 3-D input: bias broadcasts over all leading dims
    x3 = x.view(4, 16, 256).to(device)
    assert torch.equal(onn.fused_bias_gelu(x3, bd.detach()).view(64, 256), y.detach())
    y0 = onn.fused_gelu(xd.detach())
    check(y0, f64(torch.nn.functional.gelu(x.double(), approximate="tanh")), "fused_gelu", atol=1e-6)


def test_fused_bias_dropout_module(device):
    m = onn.FusedBiasDropout(p=0.25).to(device)
    assert m.p == 0.25 and m.training and not m.inplace
    x = randn((128, 512), BF16, 1).to(device).requires_grad_()
    b = randn((512,), BF16, 2, std=0.1).to(device).requires_grad_()
    res = randn((128, 512), BF16, 3).to(device).requires_grad_()
    torch.manual_seed(99)
    y1 = m(x, b)
    torch.manual_seed(99)
    y2 = m(x, b)
    assert torch.equal(y1, y2), "same torch seed must give the same mask"
    y3 = m(x, b)
    assert not torch.equal(y1, y3), "consecutive calls must draw different masks"
    # the mask is Philox with torch's seed and the generator offset at the call
    from oslo_amd.torch import _C

    kept = _C.get_fused_elementwise_kernel().philox_mask(128 * 512, 0.25, 99, 0, device)
    kept = kept.view(128, 512).bool()
    assert abs(kept.float().mean().item() - 0.75) < 0.02
    assert (y1[~kept] == 0).all()
    want = ((x.detach().float() + b.detach().float()) / 0.75)[kept]
    assert torch.allclose(y1.float()[kept], want, rtol=2 ** -7)
    # backward regenerates the same mask
    g = randn((128, 512), BF16, 4).to(device)
    y1.backward(g)
    assert torch.equal(x.grad == 0, ~kept | (g == 0))
    assert b.grad.shape == (512,)
    # fused residual add
    x.grad = None
    torch.manual_seed(99)
    y4 = m(x, b, res)
    assert (y4.float() - (y1.float() + res.float())).abs().max() <= 2 ** -4
    y4.backward(g)
    assert torch.equal(res.grad, g)
    # eval mode: plain x + bias
    m.eval()
    ye = m(x, b)
    assert torch.equal(ye, (x.float() + b.float()).to(BF16))


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("mask_type", ["causal", "padding"])
def test_fused_scale_mask_softmax_module(device, dtype, mask_type):
    b, h, sq, sk = 2, 4, 64, 64
    x = randn((b, h, sq, sk), dtype, 1, std=2.0)
    g = randn((b, h, sq, sk), dtype, 2)
    kwargs = dict(
        input_in_fp16=dtype == F16, input_in_bf16=dtype == BF16, softmax_in_fp32=True, scale=0.125,
        attn_mask_type=onn.AttnMaskType.causal if mask_type == "causal" else onn.AttnMaskType.padding,
    )
    fused = onn.FusedScaleMaskSoftmax(scaled_masked_softmax_fusion=True, **kwargs)
    unfused = onn.FusedScaleMaskSoftmax(scaled_masked_softmax_fusion=False, **kwargs)
    mask = None
    if mask_type == "padding":
        valid = torch.tensor([64, 40])
        mask = (torch.arange(sk)[None, :] >= valid[:, None]).view(b, 1, 1, sk)
    xd = x.to(device).requires_grad_()
    md = None if mask is None else mask.to(device)
    assert fused.is_kernel_available(md, b, h, sq, sk, input=xd)
    y = fused(xd, md)
    y.backward(g.to(device))
    xr = x.double().requires_grad_()
    ref_mod = onn.FusedScaleMaskSoftmax(scaled_masked_softmax_fusion=False, scale=0.125,
                                        attn_mask_type=kwargs["attn_mask_type"])
    yr = ref_mod(xr, mask)
    yr.backward(g.double())
    assert y.dtype == dtype
    check(y, f64(yr), "FusedScaleMaskSoftmax fwd", atol=1e-9)
    # the float64 gradient flows through the unrounded probabilities; the fused
    # backward starts from the stored (rounded) ones: compare at that precision
    tol = {F32: 1e-5, F16: 2e-3, BF16: 1.6e-2}[dtype]
    err = (xd.grad.double().cpu() - xr.grad).abs().max().item()
    assert err <= tol * xr.grad.abs().max().item() + 1e-7, err
    # unfused branch on the GPU agrees with the fused one
    yu = unfused(x.to(device), md)
    assert (yu.float() - y.detach().float()).abs().max() <= (2 ** -8 if dtype != F32 else 1e-6)
    # CPU tensors take the unfused branch
    assert not fused.is_kernel_available(mask, b, h, sq, sk, input=x)
    yc = fused(x, mask)
    assert yc.device.type == "cpu"


def test_fused_scale_mask_softmax_adds_a_floating_point_mask(device):
    """A floating-point mask is an additive term (it may carry finite biases):
    the fused branch computes softmax(scale * x + mask), never "masked out or
    not"; a mask on another device leaves the call to the torch chain."""
    b, h, sq, sk = 2, 3, 16, 32
    x = randn((b, h, sq, sk), F32, 5).to(device)
    bias = randn((b, 1, sq, sk), F32, 6).to(device)
    m = onn.FusedScaleMaskSoftmax(scale=0.5)
    assert m.is_kernel_available(bias, b, h, sq, sk, input=x)
    assert torch.allclose(m(x, bias), torch.softmax(0.5 * x + bias, dim=-1), rtol=1e-5, atol=1e-7)
    assert not m.is_kernel_available(torch.zeros(b, 1, 1, sk, dtype=torch.bool), b, h, sq, sk, input=x)
    assert not m.is_kernel_available(torch.zeros(b, 1, 1, sk + 1, device=device), b, h, sq, sk, input=x)


def test_fused_scale_mask_softmax_without_a_mask_and_with_an_integer_mask(device):
    """A padding-type module called without a mask is a plain scaled softmax; a
    mask of integers counts as its non-zero pattern; both on the kernels (the
    torch chain would warn)."""
    import warnings

    x = randn((2, 3, 9, 64), torch.bfloat16, 5).to(device)
    m = onn.FusedScaleMaskSoftmax(input_in_bf16=True, attn_mask_type=onn.AttnMaskType.padding, scale=0.25)
    pad = torch.zeros(2, 1, 1, 64, dtype=torch.int32, device=device)
    pad[1, ..., 50:] = 7
    with warnings.catch_warnings():
        warnings.simplefilter("error", RuntimeWarning)
        y0 = m(x, None)
        y1 = m(x, pad)
    ref0 = torch.softmax(x.float() * 0.25, dim=-1)
    ref1 = torch.softmax((x.float() * 0.25).masked_fill(pad.bool(), float("-inf")), dim=-1)
    assert (y0.float() - ref0).abs().max().item() <= 4e-3 and (y1.float() - ref1).abs().max().item() <= 4e-3
    assert (y1[1, ..., 50:] == 0).all()
    # rows per workgroup of the masked kernel, as the reference's shim reports it
    # (FusedScaleMaskSoftmaxBinder.cpp:122-127)
    assert onn.FusedScaleMaskSoftmax.get_batch_per_block(9, 64, 2, 3) >= 1


def test_skip_bias_add_producers_feed_the_fused_ops(device):
    lin = onn.Linear(32, 64, skip_bias_add=True).to(device)
    conv = onn.Conv1D(64, 32, skip_bias_add=True).to(device)
    x = randn((4, 8, 32), F32, 1).to(device)
    out, bias = lin(x)
    assert out.shape == (4, 8, 64) and bias is lin.bias
    y = onn.fused_bias_gelu(out, bias)
    ref = torch.nn.functional.gelu(torch.nn.functional.linear(x, lin.weight, lin.bias), approximate="tanh")
    assert torch.allclose(y, ref, rtol=1e-4, atol=1e-5)
    out, bias = conv(x)
    assert out.shape == (4, 8, 64) and bias is conv.bias
    drop = onn.FusedBiasDropout(0.0).to(device)
    assert torch.allclose(drop(out, bias), out + bias)
