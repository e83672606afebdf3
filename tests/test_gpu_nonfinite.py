"""Non-finite inputs on the GPU: an inf or a NaN poisons its own row (norms,
softmax) or its own element (bias-GeLU, bias-dropout-add) exactly as it does in
the reference's unfused torch path, and leaves every other row bit-identical to
the run without it."""
import pytest
import torch

from helpers import randn
from oracle import torch_path as tp
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

BF16, F32 = torch.bfloat16, torch.float32
BAD = [float("inf"), float("-inf"), float("nan")]


def _same_nan_pattern(a, ref):
    a, ref = a.float().cpu(), ref.float().cpu()
    assert torch.equal(torch.isnan(a), torch.isnan(ref)), "NaN pattern differs"
    assert torch.equal(torch.isinf(a), torch.isinf(ref)), "inf pattern differs"
    assert torch.equal(torch.sign(a[torch.isinf(ref)]), torch.sign(ref[torch.isinf(ref)]))


@pytest.mark.parametrize("bad", BAD)
@pytest.mark.parametrize("dtype,n2", [(BF16, 4096), (F32, 1024), (BF16, 128), (BF16, 100)])
def test_norms(device, bad, dtype, n2):
    n1 = 24
    x = randn((n1, n2), dtype, seed=1)
    gamma = randn((n2,), dtype, seed=2, std=0.02, mean=1.0)
    beta = randn((n2,), dtype, seed=3, std=0.02)
    dy = randn((n1, n2), dtype, seed=4)
    xb = x.clone()
    xb[5, 17] = bad
    k = _C.get_layernorm_kernel()
    outs = []
    for t in (x, xb):
        td = t.to(device)
        y, mean, invvar = k.layer_norm_forward_affine(td, (n2,), gamma.to(device), beta.to(device), 1e-5)
        dx, dg, db = k.layer_norm_backward_affine(dy.to(device), mean, invvar, td, (n2,),
                                                  gamma.to(device), beta.to(device), 1e-5)
        r, rinv = k.rms_norm_forward_affine(td, (n2,), gamma.to(device), 1e-5)
        rdx, rdg = k.rms_norm_backward_affine(dy.to(device), rinv, td, (n2,), gamma.to(device), 1e-5)
        outs.append((y, dx, r, rdx))
    ref_ln = tp.layer_norm(xb.float(), gamma.float(), beta.float(), 1e-5)
    ref_rms = tp.rms_norm(xb.float(), gamma.float(), 1e-5)
    good = torch.arange(n1) != 5
    for clean, dirty, ref in zip(outs[0], outs[1], (ref_ln, None, ref_rms, None)):
        # every other row: bit-identical to the clean run
        assert torch.equal(clean[good], dirty[good])
        if ref is not None:
            _same_nan_pattern(dirty, ref)
    # forward of the poisoned row, spelled out: all NaN for LayerNorm
    assert torch.isnan(outs[1][0][5].float()).all()


@pytest.mark.parametrize("bad", BAD)
def test_bias_gelu_and_bias_dropout_add(device, bad):
    n1, n2 = 16, 1024
    x = randn((n1, n2), BF16, seed=5)
    b = randn((n2,), BF16, seed=6, std=0.1)
    res = randn((n1, n2), BF16, seed=7)
    xb = x.clone()
    xb[3, 9] = bad
    k = _C.get_fused_elementwise_kernel()
    y0 = k.bias_gelu_forward(x.to(device), b.to(device))
    y1 = k.bias_gelu_forward(xb.to(device), b.to(device))
    ref = tp.bias_gelu(xb.float(), b.float())
    _same_nan_pattern(y1, ref)
    keep = torch.ones(n1, n2, dtype=torch.bool)
    keep[3, 9] = False
    assert torch.equal(y0.cpu()[keep], y1.cpu()[keep])
    o0 = k.bias_dropout_add_forward(x.to(device), b.to(device), res.to(device), 0.0, 1, 0)
    o1 = k.bias_dropout_add_forward(xb.to(device), b.to(device), res.to(device), 0.0, 1, 0)
    ref = xb.float() + b.float() + res.float()
    _same_nan_pattern(o1, ref)
    assert torch.equal(o0.cpu()[keep], o1.cpu()[keep])


@pytest.mark.parametrize("bad", BAD)
@pytest.mark.parametrize("sk", [1024, 128, 100])
def test_softmax(device, bad, sk):
    ab, sq = 3, sk
    x = randn((ab, sq, sk), BF16, seed=8)
    xb = x.clone()
    xb[1, sq - 1, 3] = bad          # the last query sees every key
    k = _C.get_softmax_kernel()
    y0 = k.fused_scaled_upper_triang_masked_softmax_forward(x.to(device), 0.5)
    y1 = k.fused_scaled_upper_triang_masked_softmax_forward(xb.to(device), 0.5)
    ref = tp.causal_softmax(xb.float(), 0.5)
    _same_nan_pattern(y1, ref)
    good = torch.ones(ab, sq, dtype=torch.bool)
    good[1, sq - 1] = False
    assert torch.equal(y0.cpu()[good], y1.cpu()[good])
    # a key beyond the diagonal is never read: poison there changes nothing
    xc = x.clone()
    xc[1, 2, sk - 1] = bad
    y2 = k.fused_scaled_upper_triang_masked_softmax_forward(xc.to(device), 0.5)
    assert torch.equal(y0, y2)
