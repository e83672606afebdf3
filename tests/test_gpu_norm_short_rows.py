"""LayerNorm / RMSNorm on short rows on the GPU: rows of at most 32 chunks
(256 16-bit elements, 128 fp32 elements) lie side by side in a wavefront, 8, 16
or 32 lanes each.  Every lane-group size runs here, forward and backward, with
ragged and full rows, against the float64 oracle (same checks and tolerances
as tests/test_gpu_norm.py), and against one row per wavefront."""
import pytest
import torch

import test_gpu_norm as base
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

# (n2, input dtype, output dtype); chunks = n2 / 8 (16-bit) or n2 / 4 (fp32 input)
ROWS = [
    (8, BF16, BF16), (24, F16, F16), (64, BF16, BF16),        # <= 8 chunks
    (72, F16, F16), (128, BF16, BF16),                        # <= 16 chunks
    (136, BF16, BF16), (200, F16, F16), (256, BF16, BF16),    # <= 32 chunks
    (4, F32, F32), (32, F32, F32), (36, F32, F32), (64, F32, F32),
    (100, F32, F32), (128, F32, F32),
    (64, F32, BF16), (128, F32, F16),                         # fp32 input, 16-bit output
    # exactly 3 x 8 / 16 / 32 chunks: three chunks per lane, rows side by side
    (192, BF16, BF16), (384, F16, F16), (768, BF16, BF16), (768, F16, F16),
    (96, F32, F32), (192, F32, F32), (384, F32, F32), (768, F32, BF16),
]
N1 = [1, 37, 5003]


@pytest.fixture
def tuned():
    yield
    _C.tune("norm_lanes_per_row", 0)


# a non-affine norm returns the input's dtype, so it runs where tin == tout
SHORT_CASES = [(n2, tin, tout, n1, affine) for (n2, tin, tout) in ROWS for n1 in N1
               for affine in (True, False) if affine or tin == tout]


@pytest.mark.parametrize("n2,tin,tout,n1,affine", SHORT_CASES)
def test_short_rows(device, tuned, n2, tin, tout, n1, affine):
    base.test_layer_norm(device, n1, n2, tin, tout, affine)
    base.test_rms_norm(device, n1, n2, tin, tout, affine)


@pytest.mark.parametrize("lanes", [16, 32, 64])
@pytest.mark.parametrize("n2,tin,tout", [(40, BF16, BF16), (64, F16, F16), (20, F32, F32)])
def test_wider_lane_groups_than_needed(device, tuned, n2, tin, tout, lanes):
    # the same rows in wider lane groups (spare lanes idle) and one per wavefront
    _C.tune("norm_lanes_per_row", lanes)
    base.test_layer_norm(device, 777, n2, tin, tout, True)
    base.test_rms_norm(device, 777, n2, tin, tout, True)


def test_side_by_side_agrees_with_one_row_per_wavefront(device, tuned):
    k = _C.get_layernorm_kernel()
    n1, n2 = 3001, 128
    x, gamma, beta, dy = (t.to(device) for t in base.make_inputs(n1, n2, BF16, BF16, seed=5))
    outs = []
    for lanes in (0, 64):
        _C.tune("norm_lanes_per_row", lanes)
        y, mean, invvar = k.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
        dx, dg, db = k.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, 1e-5)
        r, rinv = k.rms_norm_forward_affine(x, (n2,), gamma, 1e-5)
        rdx, rdg = k.rms_norm_backward_affine(dy, rinv, x, (n2,), gamma, 1e-5)
        outs.append((y, mean, invvar, dx, dg, db, r, rinv, rdx, rdg))
    for a, b in zip(*outs):
        # different summation orders: fp32 statistics agree to a few ulp, the
        # 16-bit results round to the same value almost everywhere
        af, bf = a.float(), b.float()
        if a.dtype == F32:
            assert torch.allclose(af, bf, rtol=1e-5, atol=1e-6)
        else:
            assert torch.allclose(af, bf, rtol=2e-2, atol=1e-2)
            assert (af == bf).float().mean() > 0.97
