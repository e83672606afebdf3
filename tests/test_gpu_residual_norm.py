"""Bias + dropout + residual add fused into LayerNorm / RMSNorm, forward and
backward on the GPU through the C ABI: against the float64 oracle with the
Philox oracle's keep mask, and bit for bit against the composition of the plain
entry points it replaces."""
import numpy as np
import pytest
import torch

from helpers import NP_NAME, check, f64, randn
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

CASES = [
    # (n1, n2, dtype, p)
    (64, 4096, BF16, 0.1),      # config-2/4 row length: two chunks per lane
    (48, 6144, BF16, 0.1),      # config-5 row length: three waves of four chunks
    (33, 8192, F16, 0.1),
    (20, 1024, F32, 0.1),       # 4-element chunks: half a Philox group each
    (17, 4096, F32, 0.2),
    (50, 768, F16, 0.1),        # BERT-base hidden size
    (9, 520, BF16, 0.3),        # ragged: 65 chunks
    (40, 64, BF16, 0.1),
    (5, 16384, BF16, 0.1),      # up to 1024 threads per row
    (3, 12288, F16, 0.1),
    (7, 100, F32, 0.1),         # vector path needs n2 % 4 == 0: ok; 25 chunks
    (6, 1001, BF16, 0.1),       # odd length: composed scalar path
    (4, 40000, BF16, 0.1),      # beyond the register path: composed path
    # short rows side by side in a wavefront (8 / 16 / 32 lanes per row)
    (1003, 256, BF16, 0.1),
    (517, 128, F16, 0.2),
    (2050, 64, BF16, 0.1),
    (333, 40, BF16, 0.1),       # 5 chunks in 8 lanes
    (700, 100, F32, 0.1),       # 25 fp32 chunks in 32 lanes
    (90, 7168, BF16, 0.1),      # 16 elements per lane over seven waves
    (1001, 768, BF16, 0.1),     # three chunks per lane, two rows per wave
    (515, 384, F16, 0.2),
    (260, 192, BF16, 0.1),
    (300, 384, F32, 0.1),
    (1, 8, F32, 0.5),
    (12, 2048, BF16, 0.0),      # no dropout
    (12, 2048, BF16, 1.0),      # everything dropped
]


def make_inputs(n1, n2, dtype, seed):
    x = randn((n1, n2), dtype, seed)
    res = randn((n1, n2), dtype, seed + 1)
    bias = randn((n2,), dtype, seed + 2, std=0.1)
    gamma = randn((n2,), dtype, seed + 3, std=0.1, mean=1.0)
    beta = randn((n2,), dtype, seed + 4, std=0.1)
    dy = randn((n1, n2), dtype, seed + 5)
    dh = randn((n1, n2), dtype, seed + 6)
    return x, res, bias, gamma, beta, dy, dh


@pytest.mark.parametrize("rms", [False, True])
@pytest.mark.parametrize("n1,n2,dtype,p", CASES)
def test_fused_vs_oracle(device, n1, n2, dtype, p, rms):
    seed, offset = 4321 + n2, 4 * n1
    x, res, bias, gamma, beta, dy, dh = make_inputs(n1, n2, dtype, n1 + n2)
    k = _C.get_layernorm_kernel()
    eps = 1e-5
    name = NP_NAME[dtype]
    y, h, mean, invvar = k.bias_dropout_add_norm_forward(
        rms, x.to(device), bias.to(device), res.to(device), (n2,), gamma.to(device),
        None if rms else beta.to(device), eps, p, seed, offset,
    )
    keep = philox.keep_mask(n1 * n2, p, seed, offset).reshape(n1, n2).astype(bool)
    # h against the unrounded oracle (the kernel's fp32 evaluation can land on the
    # other side of a rounding tie); y and the statistics from the h the kernel stored
    check(h, cf.bias_dropout_add_fwd(f64(x), f64(bias), f64(res), keep, p), "fused fwd h", atol=1e-6)
    assert (h.cpu()[torch.from_numpy(~keep)] == res[torch.from_numpy(~keep)]).all()
    if rms:
        oy, oinv = cf.rms_norm_fwd(f64(h), f64(gamma), eps, name)
        omean = None
    else:
        oy, omean, oinv = cf.layer_norm_fwd(f64(h), f64(gamma), f64(beta), eps, name)
    check(y, oy, "fused fwd y", atol=1e-6, max_ulp=2 if rms else 1)
    assert np.allclose(f64(invvar), oinv, rtol=2e-6)
    if not rms:
        assert np.allclose(f64(mean), omean, rtol=1e-5, atol=1e-6)
    # backward from the kernel's own saved h / statistics
    g_res, g_in, g_gamma, g_beta, g_bias = k.bias_dropout_add_norm_backward(
        rms, dy.to(device), dh.to(device), h, mean, invvar, (n2,), gamma.to(device),
        p, seed, offset,
    )
    odres, odx, odg, odb, odbias = cf.bias_dropout_add_norm_bwd(
        f64(dy), f64(dh), f64(h), None if rms else f64(mean), f64(invvar), f64(gamma), keep, p, rms, name
    )
    check(g_res, odres, "fused bwd dres", atol=2e-6)
    check(g_in, odx, "fused bwd dx", atol=2e-6)
    if p > 0:
        assert (g_in.cpu()[torch.from_numpy(~keep)] == 0).all()
    else:
        assert g_in.data_ptr() == g_res.data_ptr()
    col_scale = float(np.sqrt(n1))
    check(g_gamma, odg, "fused bwd dgamma", atol=1e-5 * col_scale, max_ulp=2)
    if not rms:
        check(g_beta, odb, "fused bwd dbeta", atol=1e-5 * col_scale, max_ulp=2)
    # dbias: column sums of dx as the kernel stored it
    want = f64(g_in).sum(0)
    check(g_bias, want, "fused bwd dbias", atol=1e-5 * col_scale, max_ulp=2)


@pytest.mark.parametrize("n1,n2,dtype", [(64, 4096, BF16), (30, 6144, BF16), (20, 1024, F32), (9, 520, F16), (6, 1001, BF16)])
def test_fused_equals_composition_of_plain_entry_points(device, n1, n2, dtype):
    """h of the fused forward is bit-identical to oslo_bias_dropout_add_fwd and y
    is oslo_ln_fwd of it (to the last place); with no second consumer of h and
    p = 0 the fused backward's dres is bit-identical to oslo_ln_bwd's dx."""
    p, seed, offset = 0.1, 77, 40
    x, res, bias, gamma, beta, dy, dh = [t.to(device) for t in make_inputs(n1, n2, dtype, 3)]
    k = _C.get_layernorm_kernel()
    ek = _C.get_fused_elementwise_kernel()
    y, h, mean, invvar = k.bias_dropout_add_norm_forward(
        False, x, bias, res, (n2,), gamma, beta, 1e-5, p, seed, offset
    )
    h2 = ek.bias_dropout_add_forward(x, bias, res, p, seed, offset)
    y2, mean2, invvar2 = k.layer_norm_forward_affine(h2, (n2,), gamma, beta, 1e-5)
    assert torch.equal(h, h2)
    # (the fused kernel may split a row over the waves differently: the
    # statistics can then differ in the last bit and y in a rare last place)
    assert torch.allclose(mean, mean2, rtol=1e-5, atol=1e-7) and torch.allclose(invvar, invvar2, rtol=2e-6)
    differ = y != y2
    assert int(differ.sum()) <= max(3, 1e-3 * y.numel()) or y.dtype == torch.float32
    rel = 1e-5 if y.dtype == torch.float32 else 2.0 ** -7
    assert ((y.float() - y2.float()).abs() <= rel * y2.float().abs() + 1e-5).all()
    # without h_out the same y
    y3, h3, _, _ = k.bias_dropout_add_norm_forward(
        False, x, bias, res, (n2,), gamma, beta, 1e-5, p, seed, offset, want_h=False
    )
    assert h3 is None and torch.equal(y3, y)
    g_res, g_in, g_gamma, g_beta, g_bias = k.bias_dropout_add_norm_backward(
        False, dy, None, h, mean, invvar, (n2,), gamma, 0.0, 0, 0
    )
    dx2, dg2, db2 = k.layer_norm_backward_affine(dy, mean, invvar, h, (n2,), gamma, beta, 1e-5)
    assert torch.equal(g_res, dx2) and torch.equal(g_gamma, dg2) and torch.equal(g_beta, db2)


def test_optional_operands_and_argument_checks(device):
    n1, n2 = 10, 256
    x, res, bias, gamma, beta, dy, dh = [t.to(device) for t in make_inputs(n1, n2, BF16, 9)]
    k = _C.get_layernorm_kernel()
    # no bias, no residual, no affine: plain LayerNorm of x
    y, h, mean, invvar = k.bias_dropout_add_norm_forward(
        False, x, None, None, (n2,), None, None, 1e-5, 0.0, 0, 0
    )
    y2, _, _ = k.layer_norm_forward(x, (n2,), 1e-5)
    assert torch.equal(h, x) and torch.equal(y, y2)
    g_res, g_in, g_gamma, g_beta, g_bias = k.bias_dropout_add_norm_backward(
        False, dy, None, h, mean, invvar, (n2,), None, 0.0, 0, 0, need_bias_grad=False
    )
    assert g_gamma is None and g_beta is None and g_bias is None
    assert torch.equal(g_res, k.layer_norm_backward(dy, mean, invvar, x, (n2,), 1e-5))
    with pytest.raises(RuntimeError):
        k.bias_dropout_add_norm_forward(False, x, bias.float(), res, (n2,), gamma, beta, 1e-5, 0.1, 0, 0)
    with pytest.raises(RuntimeError):
        k.bias_dropout_add_norm_forward(False, x, bias, res[:5], (n2,), gamma, beta, 1e-5, 0.1, 0, 0)
    with pytest.raises(RuntimeError):
        k.bias_dropout_add_norm_forward(False, x, bias, res, (n2,), gamma, beta, 1e-5, 1.5, 0, 0)


@pytest.mark.parametrize("rms", [False, True])
def test_module_and_autograd(device, rms):
    """The module against the reference's chain of modules on the same Philox
    state: FusedBiasDropout -> add -> (Fused)LayerNorm, gradients of every
    operand, and a second consumer of the residual sum (pre-LN block)."""
    import oslo_amd.torch.nn as onn

    n1, n2, p = 96, 1024, 0.1
    x, res, bias, gamma, beta, dy, dh = make_inputs(n1, n2, BF16, 21)
    cls = onn.FusedBiasDropoutAddRMSNorm if rms else onn.FusedBiasDropoutAddLayerNorm
    m = cls(n2, p=p, eps=1e-5, return_sum=True).to(device).to(BF16)
    with torch.no_grad():
        m.weight.copy_(gamma)
        if not rms:
            m.bias.copy_(beta)
    leaves = [t.to(device).requires_grad_(True) for t in (x, bias, res)]
    torch.manual_seed(11)
    gen = torch.cuda.default_generators[leaves[0].device.index or 0]
    seed, offset = gen.initial_seed(), gen.get_offset()
    y, h = m(*leaves)
    assert gen.get_offset() == offset + 4
    # one backward with both consumers of h: autograd hands grad_y and grad_h
    # to the fused backward together
    ((y * dy.to(device)).sum() + (h * dh.to(device)).sum()).backward()
    keep = philox.keep_mask(n1 * n2, p, seed, offset).reshape(n1, n2).astype(bool)
    check(h, cf.bias_dropout_add_fwd(f64(x), f64(bias), f64(res), keep, p), "module h", atol=1e-6)
    hk = f64(h)
    if rms:
        oy, oinv = cf.rms_norm_fwd(hk, f64(gamma), 1e-5, "bf16")
        omean = None
    else:
        oy, omean, oinv = cf.layer_norm_fwd(hk, f64(gamma), f64(beta), 1e-5, "bf16")
    check(y, oy, "module y", atol=1e-6, max_ulp=2 if rms else 1)
    odres, odx, odg, odb, odbias = cf.bias_dropout_add_norm_bwd(
        f64(dy), f64(dh), hk, omean, oinv, f64(gamma), keep, p, rms, "bf16"
    )
    check(leaves[2].grad, odres, "module dres", atol=2e-6)
    check(leaves[0].grad, odx, "module dx", atol=2e-6)
    check(leaves[1].grad, f64(leaves[0].grad).sum(0), "module dbias", atol=1e-4, max_ulp=2)
    check(m.weight.grad, odg, "module dgamma", atol=1e-4, max_ulp=2)
    if not rms:
        check(m.bias.grad, odb, "module dbeta", atol=1e-4, max_ulp=2)
    # eval mode: no dropout, generator untouched
    m.eval()
    off = gen.get_offset()
    y_eval, h_eval = m(*[t.detach() for t in leaves])
    assert gen.get_offset() == off
    check(h_eval, cf.bias_dropout_add_fwd(f64(x), f64(bias), f64(res), None, 0.0), "module eval h", atol=1e-6)
    if rms:
        oy0, _ = cf.rms_norm_fwd(f64(h_eval), f64(gamma), 1e-5, "bf16")
    else:
        oy0, _, _ = cf.layer_norm_fwd(f64(h_eval), f64(gamma), f64(beta), 1e-5, "bf16")
    check(y_eval, oy0, "module eval y", atol=1e-6, max_ulp=2 if rms else 1)


@pytest.mark.parametrize("n1,n2,dtype,rms,second", [
    (48, 16384, BF16, False, True), (40, 14336, F16, False, False), (24, 12288, F32, False, True),
    (48, 16384, BF16, True, False), (16, 8192, F32, True, True),
])
def test_wide_rows_take_the_two_backward_kernels(device, monkeypatch, n1, n2, dtype, rms, second):
    """Rows beyond 12288 16-bit or 6144 float32 elements: the module's backward
    runs the norm's backward kernel and then the bias-dropout-add backward
    kernel (the one-kernel backward spills there).  Gradients against the
    float64 oracle; the gradient of the sum is rounded to its dtype between
    the two kernels, as in the chain of unfused modules, so 16-bit results may
    differ from the one-kernel oracle by an ulp more often."""
    import oslo_amd.torch.nn as onn
    from oslo_amd.torch import _C

    p = 0.1
    x, res, bias, gamma, beta, dy, dh = make_inputs(n1, n2, dtype, 31)
    kernel = _C.get_layernorm_kernel()
    fused_calls = []
    real = kernel.bias_dropout_add_norm_backward
    monkeypatch.setattr(kernel, "bias_dropout_add_norm_backward",
                        lambda *a, **k: fused_calls.append(1) or real(*a, **k))
    leaves = [t.to(device).requires_grad_(True) for t in (x, bias, res)]
    w = gamma.to(device).requires_grad_(True)
    b = None if rms else beta.to(device).requires_grad_(True)
    torch.manual_seed(5)
    gen = torch.cuda.default_generators[leaves[0].device.index or 0]
    seed, offset = gen.initial_seed(), gen.get_offset()
    if rms:
        y, h = onn.fused_bias_dropout_add_rms_norm(*leaves, w, (n2,), 1e-5, p, True, return_sum=True)
    else:
        y, h = onn.fused_bias_dropout_add_layer_norm(*leaves, w, b, (n2,), 1e-5, p, True, return_sum=True)
    loss = (y * dy.to(device)).sum()
    if second:
        loss = loss + (h * dh.to(device)).sum()
    loss.backward()
    assert not fused_calls, "the one-kernel backward ran"
    keep = philox.keep_mask(n1 * n2, p, seed, offset).reshape(n1, n2).astype(bool)
    name = NP_NAME[dtype]
    hk = f64(h)
    if rms:
        _, oinv = cf.rms_norm_fwd(hk, f64(gamma), 1e-5, name)
        omean = None
    else:
        _, omean, oinv = cf.layer_norm_fwd(hk, f64(gamma), f64(beta), 1e-5, name)
    odres, odx, odg, odb, _ = cf.bias_dropout_add_norm_bwd(
        f64(dy), f64(dh) if second else None, hk, omean, oinv, f64(gamma), keep, p, rms, name)
    lowp = dict(max_ulp=2, min_exact=0.9) if dtype != F32 else {}
    # (the norm's gradient is rounded before the second consumer's gradient is added:
    #  half an ulp of that operand is the absolute error of a sum that cancels)
    floor = 4e-6
    if second and dtype != F32:
        floor = 0.5 * float(torch.finfo(dtype).eps) * float(np.abs(odres).max() + np.abs(f64(dh)).max())
    check(leaves[2].grad, odres, "wide dres", atol=floor, **lowp)
    # (dx = keep * round(dres) / (1 - p) is rounded twice: a quarter of the 16-bit values land an ulp
    #  beside the once-rounded oracle)
    if dtype != F32:
        lowp = dict(max_ulp=2, min_exact=0.7, l2_tol=4e-3)
    check(leaves[0].grad, odx, "wide dx", atol=floor / (1 - p), **lowp)
    col = 1e-5 * np.sqrt(n1) + 1e-6
    check(leaves[1].grad, f64(leaves[0].grad).sum(0), "wide dbias", atol=3 * col, max_ulp=2, min_exact=0.97)
    check(w.grad, odg, "wide dgamma", atol=3 * col, max_ulp=2, min_exact=0.97)
    if not rms:
        check(b.grad, odb, "wide dbeta", atol=col, max_ulp=2, min_exact=0.97)


def test_unused_outputs_get_no_materialised_gradient(device, monkeypatch):
    """A post-LN block uses y only: backward must hand the kernel no dh_extra
    (not a zero-filled tensor, which costs a fill and a full read).  A caller
    that uses h only gets the backward of dropout(x + bias) + residual."""
    import oslo_amd.torch.nn as onn
    from oslo_amd.torch import _C

    n1, n2, p = 64, 512, 0.1
    x, res, bias, gamma, beta, dy, dh = make_inputs(n1, n2, BF16, 5)
    seen = []
    kernel = _C.get_layernorm_kernel()
    real = kernel.bias_dropout_add_norm_backward

    def spy(rms, grad_y, grad_h, *a, **k):
        seen.append(grad_h)
        return real(rms, grad_y, grad_h, *a, **k)

    monkeypatch.setattr(kernel, "bias_dropout_add_norm_backward", spy)
    leaves = [t.to(device).requires_grad_(True) for t in (x, bias, res)]
    w, b = gamma.to(device).requires_grad_(True), beta.to(device).requires_grad_(True)
    torch.manual_seed(3)
    y = onn.fused_bias_dropout_add_layer_norm(*leaves, w, b, (n2,), 1e-5, p, True)
    (y * dy.to(device)).sum().backward()
    assert seen == [None], "the unused h must not produce a gradient tensor"
    both = [t.grad.clone() for t in leaves]
    # the same call with return_sum, h consumed with a zero weight: same gradients
    for t in leaves + [w, b]:
        t.grad = None
    torch.manual_seed(3)
    y2, h2 = onn.fused_bias_dropout_add_layer_norm(*leaves, w, b, (n2,), 1e-5, p, True, return_sum=True)
    ((y2 * dy.to(device)).sum() + (h2 * 0).sum()).backward()
    for a, t in zip(both, leaves):
        assert torch.equal(a, t.grad)
    # h only: equals bias-dropout-add's own backward on the same Philox state
    for t in leaves + [w, b]:
        t.grad = None
    torch.manual_seed(3)
    _, h3 = onn.fused_bias_dropout_add_layer_norm(*leaves, w, b, (n2,), 1e-5, p, True, return_sum=True)
    (h3 * dh.to(device)).sum().backward()
    got = [t.grad.clone() for t in leaves]
    assert w.grad is None or float(w.grad.abs().max()) == 0.0
    for t in leaves:
        t.grad = None
    torch.manual_seed(3)
    h4 = onn.fused_bias_dropout_add(*leaves, p, True)
    (h4 * dh.to(device)).sum().backward()
    assert torch.equal(h3, h4)
    for a, t in zip(got, leaves):
        assert torch.equal(a, t.grad)
