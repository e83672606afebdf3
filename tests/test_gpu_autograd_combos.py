"""The autograd layer on the GPU: every subset of inputs that requires a
gradient, gradients that arrive non-contiguous, a second backward through a
retained graph, and empty batches.  A gradient that is asked for must equal,
bit for bit, the one obtained when every input asks (the kernels are
deterministic); one that is not asked for must be None."""
import itertools

import pytest
import torch

from helpers import randn
from oslo_amd.torch.nn.modules import functional as F_

pytestmark = pytest.mark.gpu

BF16, F32 = torch.bfloat16, torch.float32
N1, N2 = 48, 256


def _inputs(device, names, dtype=BF16):
    shapes = {"x": (4, N1 // 4, N2), "res": (4, N1 // 4, N2), "b": (N2,), "w": (N2,), "nb": (N2,)}
    return {n: randn(shapes[n], dtype, seed=10 + i, std=1.0 if n in ("x", "res") else 0.1,
                     mean=1.0 if n == "w" else 0.0).to(device) for i, n in enumerate(names)}


OPS = {
    "layer_norm": (("x", "w", "nb"), lambda t: F_.fused_layer_norm_affine(t["x"], t["w"], t["nb"], (N2,), 1e-5)),
    "rms_norm": (("x", "w"), lambda t: F_.fused_rms_norm_affine(t["x"], t["w"], (N2,), 1e-5)),
    "bias_gelu": (("x", "b"), lambda t: F_.fused_bias_gelu(t["x"], t["b"])),
    "bias_dropout_add": (("x", "b", "res"),
                         lambda t: F_.fused_bias_dropout_add(t["x"], t["b"], t["res"], 0.0, True)),
    "bias_dropout_add_layer_norm": (
        ("x", "b", "res", "w", "nb"),
        lambda t: F_.fused_bias_dropout_add_layer_norm(t["x"], t["b"], t["res"], t["w"], t["nb"], (N2,),
                                                       1e-5, 0.0, True)),
    "bias_dropout_add_rms_norm": (
        ("x", "b", "res", "w"),
        lambda t: F_.fused_bias_dropout_add_rms_norm(t["x"], t["b"], t["res"], t["w"], (N2,), 1e-5, 0.0, True)),
}


def _grads(fn, base, wanted, dy):
    t = {n: v.clone().requires_grad_(n in wanted) for n, v in base.items()}
    y = fn(t)
    y.backward(dy)
    return y.detach(), {n: t[n].grad for n in t}


@pytest.mark.parametrize("op", sorted(OPS))
def test_every_subset_of_required_gradients(device, op):
    names, fn = OPS[op]
    base = _inputs(device, names)
    dy = randn((4, N1 // 4, N2), BF16, seed=99).to(device)
    y_all, g_all = _grads(fn, base, set(names), dy)
    assert all(g_all[n] is not None for n in names)
    for k in range(1, len(names)):
        for wanted in itertools.combinations(names, k):
            y, g = _grads(fn, base, set(wanted), dy)
            assert torch.equal(y, y_all)
            for n in names:
                if n in wanted:
                    assert g[n] is not None and torch.equal(g[n], g_all[n]), (op, wanted, n)
                else:
                    assert g[n] is None, (op, wanted, n)
    # nothing requires a gradient: plain forward
    with torch.no_grad():
        assert torch.equal(fn(base), y_all)


@pytest.mark.parametrize("op", sorted(OPS))
def test_non_contiguous_gradient_and_retained_graph(device, op):
    names, fn = OPS[op]
    base = _inputs(device, names)
    t = {n: v.clone().requires_grad_() for n, v in base.items()}
    y = fn(t)
    # the incoming gradient is a transposed view
    dy = randn((N1 // 4, 4, N2), BF16, seed=98).to(device).transpose(0, 1)
    assert not dy.is_contiguous()
    first = torch.autograd.grad(y, [t[n] for n in names], dy, retain_graph=True)
    second = torch.autograd.grad(y, [t[n] for n in names], dy.contiguous())
    for a, b in zip(first, second):
        assert torch.equal(a, b)


def test_softmax_functions_input_gradient_only(device):
    x = randn((6, 64, 64), BF16, seed=5).to(device)
    dy = randn((6, 64, 64), BF16, seed=6).to(device)
    for fn in (lambda t: F_.scaled_upper_triang_masked_softmax(t, 0.25),
               lambda t: F_.scaled_upper_triang_masked_softmax_dropout(t, 0.25, 0.0, True)):
        xr = x.clone().requires_grad_()
        y = fn(xr)
        g1, = torch.autograd.grad(y, xr, dy, retain_graph=True)
        g2, = torch.autograd.grad(y, xr, dy.transpose(1, 2).contiguous().transpose(1, 2))
        assert torch.equal(g1, g2)
        with torch.no_grad():
            assert torch.equal(fn(x), y.detach())
    mask = torch.zeros(2, 1, 1, 64, dtype=torch.bool, device=device)
    mask[1, ..., 40:] = True
    x4 = x.view(2, 3, 64, 64)
    xr = x4.clone().requires_grad_()
    y = F_.scaled_masked_softmax(xr, mask, 0.25)
    g, = torch.autograd.grad(y, xr, dy.view(2, 3, 64, 64))
    assert (g[1, ..., 40:] == 0).all() and torch.isfinite(g).all()


@pytest.mark.parametrize("op", sorted(OPS))
def test_empty_batch(device, op):
    names, fn = OPS[op]
    base = _inputs(device, names)
    for n in ("x", "res"):
        if n in base:
            base[n] = base[n][:0]
    t = {n: v.clone().requires_grad_() for n, v in base.items()}
    y = fn(t)
    assert y.shape == (0, N1 // 4, N2)
    y.backward(torch.empty_like(y))
    for n in names:
        assert t[n].grad is not None and t[n].grad.shape == t[n].shape
        if n not in ("x", "res"):
            assert torch.count_nonzero(t[n].grad).item() == 0
