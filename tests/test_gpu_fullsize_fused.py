"""The fused bias-dropout-add + LayerNorm op at the full size of the BASELINE
workloads it folds together (configs 4 and 5), through the C ABI: bit for bit
against the composition of the plain entry points over the whole tensor,
whole-tensor properties of the backward pass, sampled rows against the oracle."""
import math

import numpy as np
import pytest
import torch

from helpers import check, f64
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C
from test_gpu_fullsize import gpu_randn, sample_rows

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


@pytest.mark.parametrize("n1,n2", [(16384, 4096), (8192, 6144)])
def test_bias_dropout_add_layer_norm_full_size(device, n1, n2):
    seed, offset, p, eps = 1234, 0, 0.1, 1e-5
    x = gpu_randn((n1, n2), BF16, 12, device)
    res = gpu_randn((n1, n2), BF16, 13, device)
    dy = gpu_randn((n1, n2), BF16, 14, device)
    dh = gpu_randn((n1, n2), BF16, 16, device)
    bias = gpu_randn((n2,), BF16, 15, device, std=0.02)
    gamma = gpu_randn((n2,), BF16, 17, device, std=0.02, mean=1.0)
    beta = gpu_randn((n2,), BF16, 18, device, std=0.02)
    k = _C.get_layernorm_kernel()
    ek = _C.get_fused_elementwise_kernel()
    y, h, mean, invvar = k.bias_dropout_add_norm_forward(
        False, x, bias, res, (n2,), gamma, beta, eps, p, seed, offset
    )
    # forward: identical to the two plain launches over the whole tensor
    h2, mask = ek.bias_dropout_add_forward(x, bias, res, p, seed, offset, return_mask=True)
    assert torch.equal(h, h2)
    y2, mean2, invvar2 = k.layer_norm_forward_affine(h2, (n2,), gamma, beta, eps)
    # (the fused kernel may split a row over the waves differently, so the
    # statistics can differ in the last bit and y in a rare last place)
    assert torch.allclose(mean, mean2, rtol=1e-5, atol=1e-7) and torch.allclose(invvar, invvar2, rtol=2e-6)
    differ = y != y2
    assert int(differ.sum()) <= max(3, 1e-3 * y.numel()) or y.dtype == torch.float32
    rel = 1e-5 if y.dtype == torch.float32 else 2.0 ** -7
    assert ((y.float() - y2.float()).abs() <= rel * y2.float().abs() + 1e-5).all()
    del h2, y2
    # backward with a second consumer of h
    g_res, g_in, g_gamma, g_beta, g_bias = k.bias_dropout_add_norm_backward(
        False, dy, dh, h, mean, invvar, (n2,), gamma, p, seed, offset
    )
    # whole tensor: dx is zero exactly where dropped, else the residual gradient over 1 - p
    keepb = mask.bool()
    assert g_in[~keepb].count_nonzero().item() == 0
    want = g_res.float() / (1.0 - p)
    assert ((g_in.float() - want)[keepb].abs() <= 2.0 ** -7 * want[keepb].abs() + 1e-30).all()
    # the norm's own input gradient sums to ~0 over a row: sum(dres - dh_extra) ~ 0
    rowsum = (g_res.float() - dh.float()).sum(-1).abs()
    assert (rowsum <= 1.5).all()  # 4096-6144 bf16 roundings of O(1) values
    check(g_bias, g_in.double().sum(0).cpu().numpy(), "fused dbias all rows", atol=1e-5 * math.sqrt(n1), min_exact=0.97)
    # parameter gradients equal those of the plain LayerNorm backward
    _, dg2, db2 = k.layer_norm_backward_affine(dy, mean, invvar, h, (n2,), gamma, beta, eps)
    assert torch.equal(g_gamma, dg2) and torch.equal(g_beta, db2)
    # sampled rows against the oracle
    rows = sample_rows(n1, k=16)
    sel = rows.to(device)
    keep = np.stack([philox.keep_mask(n2, p, seed, offset, first_element=int(r) * n2) for r in rows]).astype(bool)
    assert np.array_equal(keep, mask[sel].cpu().numpy().astype(bool))
    odres, odx, _, _, _ = cf.bias_dropout_add_norm_bwd(
        f64(dy[sel]), f64(dh[sel]), f64(h[sel]), f64(mean[sel]), f64(invvar[sel]), f64(gamma), keep, p, False, "bf16"
    )
    check(g_res[sel], odres, "fused dres rows", atol=2e-6)
    check(g_in[sel], odx, "fused dx rows", atol=2e-6)
    oy, _, _ = cf.layer_norm_fwd(f64(h[sel]), f64(gamma), f64(beta), eps, "bf16")
    check(y[sel], oy, "fused y rows", atol=1e-6)
