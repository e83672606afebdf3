"""LayerNorm / RMSNorm forward and backward on the GPU, through the C ABI,
against the float64 oracle on identical seeded inputs.

Tolerances: fp32 outputs 1e-5 relative (plus an absolute floor for values that
cancel to ~0); 16-bit outputs at most 1 ulp from the once-rounded oracle with
>= 99.8 % bit-identical and relative L2 error <= 2e-3 (tests/helpers.py)."""
import numpy as np
import pytest
import torch

from helpers import check, check_f32, f64, randn
from oracle import closed_form as cf
from oracle import torch_path as tp
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16
NAME = {F32: "f32", F16: "f16", BF16: "bf16"}

# (n1, n2, input dtype, output/parameter dtype)
CASES = [
    (64, 4096, BF16, BF16),   # one wave or two per row, register path
    (33, 4096, BF16, BF16),   # row count not a multiple of the rows per workgroup
    (16, 6144, BF16, BF16),   # chunk count not a power of two
    (8, 8192, BF16, BF16),
    (4, 16384, F16, F16),     # several waves per row
    (3, 65536, BF16, BF16),   # largest register-resident row
    (3, 70000, BF16, BF16),   # beyond it: streaming kernel
    (7, 513, BF16, BF16),     # odd length: scalar kernel
    (3, 1, F32, F32),
    (129, 64, F16, F16),
    (1000, 32, F32, F32),
    (100, 1024, F32, F32),
    (100, 1024, F32, BF16),   # "mixed": fp32 activations, 16-bit parameters/output
    (100, 1024, F32, F16),
    (50, 768, F16, F16),
    (17, 8, BF16, BF16),
    (1, 4096, BF16, BF16),
    (300, 2048, F32, F32),
    # lengths that are no multiple of the vector width, many rows: scalar row
    # kernels and the two-step column sums through the workspace
    (3001, 100, BF16, BF16),
    (300, 4100, F16, F16),
    (2000, 37, F32, F32),
    # rows of a whole number of half-waves (96, 160, 224 chunks): the backward
    # works in units of 32 lanes
    (1003, 768, BF16, BF16),
    (517, 1280, F16, F16),
    (260, 1792, BF16, BF16),
    (129, 384, F32, F32),     # 96 fp32 chunks: whole waves
    # 16 elements per lane in the backward (part of gamma lives in LDS)
    (5, 16384, F32, F32),
    (6, 12288, F32, F32),
    (5, 16384, F32, BF16),
    (7, 12288, BF16, BF16),
    (5, 9000, F16, F16),      # ... with lanes beyond the end of the row
    (4, 14000, F32, F32),
]


# a non-affine norm returns the input's dtype, so it runs where tin == tout
AFFINE_CASES = [c + (a,) for c in CASES for a in (True, False) if a or c[2] == c[3]]


def make_inputs(n1, n2, tin, tout, seed):
    x = randn((n1, n2), tin, seed, std=1.3, mean=0.2)
    gamma = randn((n2,), tout, seed + 1, std=0.02, mean=1.0)
    beta = randn((n2,), tout, seed + 2, std=0.02)
    dy = randn((n1, n2), tout, seed + 3)
    return x, gamma, beta, dy


def stat_atol(n2):
    return 2e-6


@pytest.mark.parametrize("n1,n2,tin,tout,affine", AFFINE_CASES)
def test_layer_norm(device, n1, n2, tin, tout, affine):
    eps = 1e-5
    x, gamma, beta, dy = make_inputs(n1, n2, tin, tout, seed=n1 + n2)
    k = _C.get_layernorm_kernel()
    xd, gd, bd, dyd = (t.to(device) for t in (x, gamma, beta, dy))
    if affine:
        fwd = k.layer_norm_forward_affine_mixed_dtypes if tin != tout else k.layer_norm_forward_affine
        y, mean, invvar = fwd(xd, (n2,), gd, bd, eps)
    else:
        y, mean, invvar = k.layer_norm_forward(xd, (n2,), eps)
    assert y.dtype == tout and mean.dtype == F32 and invvar.dtype == F32
    oy, omean, oinv = cf.layer_norm_fwd(
        f64(x), f64(gamma) if affine else None, f64(beta) if affine else None, eps
    )
    check(y, oy, "ln fwd y", atol=2e-6)
    check_f32(mean, omean, "ln mean", atol=2e-6)
    check_f32(invvar, oinv, "ln invvar", atol=0)

    if affine:
        dx, dg, db = k.layer_norm_backward_affine(dyd, mean, invvar, xd, (n2,), gd, bd, eps)
    else:
        dx, dg, db = k.layer_norm_backward(dyd, mean, invvar, xd, (n2,), eps), None, None
    odx, odg, odb = cf.layer_norm_bwd(f64(dy), f64(x), omean, oinv, f64(gamma) if affine else None)
    assert dx.dtype == tin
    check(dx, odx, "ln bwd dx", atol=4e-6)
    if affine:
        assert dg.dtype == tout and db.dtype == tout
        patol = 1e-5 * np.sqrt(n1) + 1e-6
        check(dg, odg, "ln dgamma", atol=patol, min_exact=0.97)
        check(db, odb, "ln dbeta", atol=patol, min_exact=0.97)


@pytest.mark.parametrize("n1,n2,tin,tout,affine", AFFINE_CASES)
def test_rms_norm(device, n1, n2, tin, tout, affine):
    eps = 1e-5
    x, gamma, _, dy = make_inputs(n1, n2, tin, tout, seed=7 + n1 + n2)
    k = _C.get_layernorm_kernel()
    xd, gd, dyd = (t.to(device) for t in (x, gamma, dy))
    if affine:
        fwd = k.rms_norm_forward_affine_mixed_dtypes if tin != tout else k.rms_norm_forward_affine
        y, invvar = fwd(xd, (n2,), gd, eps)
    else:
        y, invvar = k.rms_norm_forward(xd, (n2,), eps)
    assert y.dtype == tout and invvar.dtype == F32
    # the oracle rounds twice (normalised value, then the product with gamma);
    # compare in the storage type.  Where fp32 vs fp64 arithmetic tips the
    # first rounding the intermediate moves by 1 ulp, and its product with a
    # gamma > 1 can then land 2 ulp away after the second rounding
    oy, oinv = cf.rms_norm_fwd(f64(x), f64(gamma) if affine else None, eps, out=NAME[tout])
    check(y, np.asarray(oy, dtype=np.float64), "rms fwd y", atol=2e-6, min_exact=0.995,
          max_ulp=2 if (affine and tout != F32) else 1)
    check_f32(invvar, oinv, "rms invvar", atol=0)

    if affine:
        dx, dg = k.rms_norm_backward_affine(dyd, invvar, xd, (n2,), gd, eps)
    else:
        dx, dg = k.rms_norm_backward(dyd, invvar, xd, (n2,), eps), None
    odx, odg = cf.rms_norm_bwd(f64(dy), f64(x), oinv, f64(gamma) if affine else None)
    check(dx, odx, "rms bwd dx", atol=4e-6)
    if affine:
        check(dg, odg, "rms dgamma", atol=1e-5 * np.sqrt(n1) + 1e-6, min_exact=0.97)


def test_unaligned_pointers_take_the_scalar_path(device):
    n1, n2 = 9, 1024
    eps = 1e-5
    base = randn((n1 * n2 + 1,), BF16, 3).to(device)
    x = base[1:].view(n1, n2)  # 2 bytes past a 16-byte boundary
    assert x.data_ptr() % 16 != 0 and x.is_contiguous()
    gamma = randn((n2,), BF16, 4, std=0.02, mean=1.0).to(device)
    beta = randn((n2,), BF16, 5, std=0.02).to(device)
    k = _C.get_layernorm_kernel()
    y, mean, invvar = k.layer_norm_forward_affine(x, (n2,), gamma, beta, eps)
    oy, omean, oinv = cf.layer_norm_fwd(f64(x), f64(gamma), f64(beta), eps)
    check(y, oy, "unaligned ln fwd")
    dy = randn((n1, n2), BF16, 6).to(device)
    dx, dg, db = k.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, eps)
    odx, odg, odb = cf.layer_norm_bwd(f64(dy), f64(x), omean, oinv, f64(gamma))
    check(dx, odx, "unaligned ln dx")
    check(dg, odg, "unaligned ln dgamma", min_exact=0.97)


def test_matches_reference_cpu_path_bf16(device):
    """Against the reference's own CPU modules (F.layer_norm / manual_rms_norm
    in bf16): bit-identical except where fp32 arithmetic order tips a rounding."""
    n1, n2, eps = 256, 4096, 1e-5
    x, gamma, beta, dy = make_inputs(n1, n2, BF16, BF16, seed=11)
    k = _C.get_layernorm_kernel()
    y, _, _ = k.layer_norm_forward_affine(x.to(device), (n2,), gamma.to(device), beta.to(device), eps)
    ref = tp.layer_norm(x, gamma, beta, eps)
    assert (y.cpu() == ref).double().mean() > 0.999
    y, _ = k.rms_norm_forward_affine(x.to(device), (n2,), gamma.to(device), eps)
    ref = tp.rms_norm(x, gamma, eps)
    assert (y.cpu() == ref).double().mean() > 0.999


def test_multi_dimensional_normalized_shape_and_leading_dims(device):
    x = randn((4, 5, 32, 16), F32, 21)
    w = randn((32, 16), F32, 22, std=0.1, mean=1.0)
    b = randn((32, 16), F32, 23, std=0.1)
    k = _C.get_layernorm_kernel()
    y, mean, invvar = k.layer_norm_forward_affine(x.to(device), (32, 16), w.to(device), b.to(device), 1e-5)
    assert y.shape == x.shape and mean.shape == (20,)
    ref = torch.nn.functional.layer_norm(x.double(), (32, 16), w.double(), b.double(), 1e-5)
    check_f32(y, ref.numpy(), "ln 2-d normalized_shape", atol=2e-6)


def test_argument_checks(device):
    k = _C.get_layernorm_kernel()
    x = torch.zeros(4, 8, device=device)
    with pytest.raises(RuntimeError, match="normalized_shape"):
        k.layer_norm_forward(x, (16,), 1e-5)
    with pytest.raises(RuntimeError, match="contiguous"):
        k.layer_norm_forward(x.t(), (4,), 1e-5)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        k.layer_norm_forward(x.cpu(), (8,), 1e-5)
    with pytest.raises(RuntimeError, match="not supported"):
        k.layer_norm_forward(x.to(torch.int32), (8,), 1e-5)
    with pytest.raises(RuntimeError, match="dtype"):
        k.layer_norm_forward_affine(x.half(), (8,), torch.ones(8, device=device), torch.zeros(8, device=device), 1e-5)
    # empty batch
    y, mean, invvar = k.layer_norm_forward(torch.zeros(0, 8, device=device), (8,), 1e-5)
    assert y.shape == (0, 8) and mean.numel() == 0
