"""LayerNorm / RMSNorm on double tensors on the GPU (the reference dispatches
double in its forward, oslo/torch/_C/csrc/fused_layer_norm.cu:780, 799, and in
the RMS backward, :950; statistics are double,
oslo/torch/_C/csrc/FusedLayerNormBinder.cpp:146-152).

Tolerance: 1e-12 relative to the output scale against the float64 oracle (both
sides compute in double; only the summation order differs).  With a double
path on the GPU, `torch.autograd.gradcheck` can pin the fused modules' backward
to finite differences of their own forward."""
import numpy as np
import pytest
import torch

from helpers import f64
from oracle import closed_form as cf
from oslo_amd.torch import _C
from oslo_amd.torch.nn import FusedLayerNorm, FusedRMSNorm
from oslo_amd.torch.nn.modules import functional as F_

pytestmark = pytest.mark.gpu

F64 = torch.float64
SHAPES = [(1, 1), (7, 1), (5, 7), (33, 513), (64, 4096), (3, 70001), (300, 64), (1030, 257)]


def _inputs(n1, n2, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((n1, n2), generator=g, dtype=F64) * 1.3 + 0.2
    gamma = 1.0 + 0.02 * torch.randn((n2,), generator=g, dtype=F64)
    beta = 0.02 * torch.randn((n2,), generator=g, dtype=F64)
    dy = torch.randn((n1, n2), generator=g, dtype=F64)
    return x, gamma, beta, dy


def _close(actual, want, what, rt=1e-12):
    a = f64(actual)
    scale = max(1.0, float(np.abs(want).max())) if want.size else 1.0
    err = float(np.abs(a - want).max()) if want.size else 0.0
    assert err <= rt * scale, "%s: max abs error %.3e (scale %.3e)" % (what, err, scale)


@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("rms", [False, True])
@pytest.mark.parametrize("n1,n2", SHAPES)
def test_f64_forward_backward(n1, n2, rms, affine, device):
    x, gamma, beta, dy = _inputs(n1, n2, 100 + n1 + n2)
    k = _C.get_layernorm_kernel()
    xd, gd, bd, dyd = (t.to(device) for t in (x, gamma, beta, dy))
    eps = 1e-5
    gn = gamma.numpy() if affine else None
    if rms:
        if affine:
            y, invvar = k.rms_norm_forward_affine(xd, (n2,), gd, eps)
        else:
            y, invvar = k.rms_norm_forward(xd, (n2,), eps)
        wy, winv = cf.rms_norm_fwd(x.numpy(), gn, eps)
        mean = None
    else:
        if affine:
            y, mean, invvar = k.layer_norm_forward_affine(xd, (n2,), gd, bd, eps)
        else:
            y, mean, invvar = k.layer_norm_forward(xd, (n2,), eps)
        wy, wmean, winv = cf.layer_norm_fwd(x.numpy(), gn, beta.numpy() if affine else None, eps)
        assert mean.dtype == F64
        _close(mean, wmean, "mean")
    assert y.dtype == F64 and invvar.dtype == F64
    _close(y, wy, "y")
    _close(invvar, winv, "invvar", rt=1e-11)

    # backward from the kernel's own statistics
    if rms:
        if affine:
            dx, dg = k.rms_norm_backward_affine(dyd, invvar, xd, (n2,), gd, eps)
        else:
            dx, dg = k.rms_norm_backward(dyd, invvar, xd, (n2,), eps), None
        wdx, wdg = cf.rms_norm_bwd(dy.numpy(), x.numpy(), f64(invvar), gn)
        db = wdb = None
    else:
        if affine:
            dx, dg, db = k.layer_norm_backward_affine(dyd, mean, invvar, xd, (n2,), gd, bd, eps)
        else:
            dx, dg, db = k.layer_norm_backward(dyd, mean, invvar, xd, (n2,), eps), None, None
        wdx, wdg, wdb = cf.layer_norm_bwd(dy.numpy(), x.numpy(), f64(mean), f64(invvar), gn)
    _close(dx, wdx, "dx", rt=1e-11)
    if affine:
        assert dg.dtype == F64
        _close(dg, wdg, "dgamma", rt=1e-11)
        if not rms:
            _close(db, wdb, "dbeta", rt=1e-11)


def test_f64_matches_torch_layer_norm_on_the_gpu(device):
    # the library routine the reference's CPU path calls
    # (oslo/torch/nn/modules/layer_norm.py:452-455), here on the same device
    x, gamma, beta, dy = (t.to(device) for t in _inputs(40, 1000, 7))
    x.requires_grad_(True)
    gamma.requires_grad_(True)
    beta.requires_grad_(True)
    want = torch.nn.functional.layer_norm(x, (1000,), gamma, beta, 1e-5)
    wgrads = torch.autograd.grad(want, (x, gamma, beta), dy)
    got = F_.fused_layer_norm_affine(x, gamma, beta, (1000,), 1e-5)
    grads = torch.autograd.grad(got, (x, gamma, beta), dy)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    for a, w in zip(grads, wgrads):
        assert torch.allclose(a, w, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape,nshape", [((6, 33), (33,)), ((2, 3, 4, 5), (4, 5))])
def test_f64_gradcheck_of_the_fused_modules(shape, nshape, device):
    torch.manual_seed(3)
    x = torch.randn(shape, dtype=F64, device=device, requires_grad=True)
    for cls in (FusedLayerNorm, FusedRMSNorm):
        for affine in (True, False):
            m = cls(nshape, eps=1e-5, elementwise_affine=affine).to(device=device, dtype=F64)
            if affine:
                with torch.no_grad():
                    for p in m.parameters():
                        p.add_(0.1 * torch.randn_like(p))
            params = tuple(m.parameters())

            def fn(inp, *ps):
                return m(inp)

            assert torch.autograd.gradcheck(fn, (x,) + params, eps=1e-6, atol=1e-6, rtol=1e-6)


def test_f64_empty_batch_and_mixed_pairs(device):
    k = _C.get_layernorm_kernel()
    x = torch.empty((0, 16), dtype=F64, device=device)
    g = torch.ones(16, dtype=F64, device=device)
    y, mean, invvar = k.layer_norm_forward_affine(x, (16,), g, g, 1e-5)
    assert y.shape == (0, 16) and mean.shape == (0,)
    dx, dg, db = k.layer_norm_backward_affine(x, mean, invvar, x, (16,), g, g, 1e-5)
    assert torch.count_nonzero(dg).item() == 0 and torch.count_nonzero(db).item() == 0
    # double activations with lower-precision parameters are not in the matrix
    x = torch.randn((4, 16), dtype=F64, device=device)
    g32 = torch.ones(16, dtype=torch.float32, device=device)
    with pytest.raises(RuntimeError):
        k.layer_norm_forward_affine_mixed_dtypes(x, (16,), g32, g32, 1e-5)
    with pytest.raises(RuntimeError):
        k.layer_norm_forward_affine_mixed_dtypes(x.float(), (16,), g, g, 1e-5)


def test_the_other_kernels_still_refuse_double(device):
    x = torch.randn((4, 16), dtype=F64, device=device)
    b = torch.zeros(16, dtype=F64, device=device)
    with pytest.raises(RuntimeError, match="float64"):
        _C.get_fused_elementwise_kernel().bias_gelu_forward(x, b)
    with pytest.raises(RuntimeError, match="float64"):
        _C.get_softmax_kernel().fused_scaled_upper_triang_masked_softmax_forward(
            x.view(1, 4, 16), 1.0)
