"""Short softmax rows on the GPU: rows of at most 32 chunks (256 16-bit keys,
128 fp32 keys) lie side by side in a wavefront, 8, 16 or 32 lanes each.  Every
lane-group size and every rows-per-wave setting of those kernels runs here,
for the causal, masked and dense forms, with and without the fused dropout,
against the float64 oracle; and the side-by-side layout must agree with one
row per wavefront up to the order of summation."""
import pytest
import torch

from helpers import check, f64, randn, ulp_distance
from oracle import closed_form as cf
from oslo_amd.torch import _C
from test_gpu_softmax import make_mask
from test_gpu_softmax_dropout import oracle_keep

pytestmark = pytest.mark.gpu


def same_up_to_summation_order(a, b):
    """Two launch shapes of one kernel add the same terms in different orders:
    the stored values agree except for rare last-place differences."""
    if a.dtype == torch.float32:
        assert torch.allclose(a, b, rtol=2e-6, atol=1e-9)
        return
    d = ulp_distance(a, b)
    assert float((d == 0).double().mean()) > 0.99
    # a last-place difference of a probability moves the gradient that is
    # computed from it; values that cancel to almost nothing differ by more
    # ulps of their own, so the bound is relative to the tensor's scale
    tol = 2.0 ** -7 * float(b.float().abs().max()) + 1e-30
    assert float((a.float() - b.float()).abs().max()) <= tol

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

# (sk, dtype): chunks per row = sk / 8 (16-bit) or sk / 4 (fp32)
LENGTHS = [
    (8, BF16), (24, F16), (64, BF16),        # <= 8 chunks
    (72, F16), (128, BF16),                  # <= 16 chunks
    (136, BF16), (200, F16), (256, BF16),    # <= 32 chunks
    (4, F32), (32, F32), (36, F32), (64, F32), (100, F32), (128, F32),
]


@pytest.fixture
def tuned():
    yield
    _C.tune("softmax_rows_per_wave", 0)
    _C.tune("softmax_lanes_per_row", 0)


@pytest.mark.parametrize("rpw", [0, 1, 2, 4])
@pytest.mark.parametrize("sk,dtype", LENGTHS)
def test_causal_short_rows(device, tuned, sk, dtype, rpw):
    ab, sq = 3, 29                      # 87 rows: no multiple of the rows per wave
    scale = 0.3
    x = randn((ab, sq, sk), dtype, seed=sk + 7)
    dy = randn((ab, sq, sk), dtype, seed=sk + 8)
    k = _C.get_softmax_kernel()
    _C.tune("softmax_rows_per_wave", rpw)
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x.to(device), scale)
    dx = k.fused_scaled_upper_triang_masked_softmax_backward(dy.to(device), y, scale)
    check(y, cf.softmax_causal_fwd(f64(x), scale), "causal fwd", atol=1e-9)
    check(dx, cf.softmax_bwd(f64(dy), f64(y), scale), "causal bwd", atol=1e-7)
    hidden = torch.from_numpy(cf.causal_hidden(sq, sk))
    has_visible = (~hidden).any(-1)
    assert (y.cpu()[:, hidden & has_visible[:, None]] == 0).all()
    # one row per wavefront: same bits
    _C.tune("softmax_lanes_per_row", 64)
    y1 = k.fused_scaled_upper_triang_masked_softmax_forward(x.to(device), scale)
    dx1 = k.fused_scaled_upper_triang_masked_softmax_backward(dy.to(device), y1, scale)
    same_up_to_summation_order(y, y1)
    same_up_to_summation_order(dx, dx1)


@pytest.mark.parametrize("kind", ["padding", "full", "rows_fully_masked", "none_masked"])
@pytest.mark.parametrize("sk,dtype", LENGTHS)
def test_masked_short_rows(device, tuned, sk, dtype, kind):
    b, np_, sq = 2, 3, 13
    scale = 0.25
    x = randn((b, np_, sq, sk), dtype, seed=sk + 1, std=2.0)
    dy = randn((b, np_, sq, sk), dtype, seed=sk + 2)
    mask = make_mask(kind, b, sq, sk, seed=sk)
    k = _C.get_softmax_kernel()
    oy = cf.softmax_masked_fwd(f64(x), mask.numpy(), scale)
    results = []
    for rpw in (1, 2, 4):
        _C.tune("softmax_rows_per_wave", rpw)
        y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), scale)
        check(y, oy, "masked fwd rpw=%d" % rpw, atol=1e-9)
        odx = cf.softmax_bwd(f64(dy), f64(y), scale)
        dx_m = k.fused_scaled_masked_softmax_backward(dy.to(device), y, scale, mask=mask.to(device))
        dx_d = k.fused_scaled_masked_softmax_backward(dy.to(device), y, scale)
        check(dx_m, odx, "masked bwd rpw=%d" % rpw, atol=1e-7)
        assert torch.equal(dx_m, dx_d)
        results.append((y, dx_m))
    full = mask.expand(b, np_, sq, sk)
    row_has_visible = (~full).any(-1, keepdim=True).expand_as(full)
    assert (results[0][0].cpu()[full & row_has_visible] == 0).all()
    for y, dx in results[1:]:
        same_up_to_summation_order(y, results[0][0])
        same_up_to_summation_order(dx, results[0][1])


@pytest.mark.parametrize("lanes", [16, 32])
def test_wider_lane_groups_than_needed(device, tuned, lanes):
    # a row of 5 chunks in a group of 16 or 32 lanes: the spare lanes stay idle
    x = randn((4, 11, 40), BF16, seed=3)
    dy = randn((4, 11, 40), BF16, seed=4)
    k = _C.get_softmax_kernel()
    y0 = k.fused_scaled_upper_triang_masked_softmax_forward(x.to(device), 0.5)
    dx0 = k.fused_scaled_upper_triang_masked_softmax_backward(dy.to(device), y0, 0.5)
    _C.tune("softmax_lanes_per_row", lanes)
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x.to(device), 0.5)
    dx = k.fused_scaled_upper_triang_masked_softmax_backward(dy.to(device), y, 0.5)
    same_up_to_summation_order(y, y0)
    same_up_to_summation_order(dx, dx0)
    check(y, cf.softmax_causal_fwd(f64(x), 0.5), "causal fwd", atol=1e-9)


@pytest.mark.parametrize("rpw", [1, 2, 4])
@pytest.mark.parametrize("sk,dtype", [(64, BF16), (128, F16), (256, BF16), (32, F32), (128, F32)])
def test_dropout_short_rows(device, tuned, sk, dtype, rpw):
    ab, sq, scale, p = 3, 21, 0.4, 0.2
    seed, offset = 77 + sk, 16
    x = randn((ab, sq, sk), dtype, seed=sk + 11)
    g = randn((ab, sq, sk), dtype, seed=sk + 12)
    k = _C.get_softmax_kernel()
    _C.tune("softmax_rows_per_wave", rpw)
    keep = oracle_keep((ab, sq, sk), p, seed, offset)
    hidden = cf.causal_hidden(sq, sk)
    out, stats = k.softmax_dropout_forward(x.to(device), None, scale, p, seed, offset)
    check(out, cf.softmax_dropout_fwd(f64(x), hidden, scale, keep, p), "dropout fwd", atol=1e-9)
    assert (out.cpu()[torch.from_numpy(~keep)] == 0).all()
    dx = k.softmax_dropout_backward(g.to(device), x.to(device), stats, None, scale, p, seed, offset)
    check(dx, cf.softmax_dropout_bwd(f64(g), f64(x), hidden, scale, keep, p), "dropout bwd", atol=2e-7)
    # masked form with a per-query mask
    b, np_ = 3, 1
    mask = make_mask("full", b, sq, sk, seed=sk)
    x4, g4 = x.view(b, np_, sq, sk), g.view(b, np_, sq, sk)
    out, stats = k.softmax_dropout_forward(x4.to(device), mask.to(device), scale, p, seed, offset)
    keep4 = keep.reshape(b, np_, sq, sk)
    check(out, cf.softmax_dropout_fwd(f64(x4), mask.numpy(), scale, keep4, p), "masked dropout fwd", atol=1e-9)
    dx = k.softmax_dropout_backward(g4.to(device), x4.to(device), stats, mask.to(device), scale, p, seed, offset)
    check(dx, cf.softmax_dropout_bwd(f64(g4), f64(x4), mask.numpy(), scale, keep4, p), "masked dropout bwd", atol=2e-7)
    # one row per wavefront: same bits
    _C.tune("softmax_lanes_per_row", 64)
    out1, stats1 = k.softmax_dropout_forward(x4.to(device), mask.to(device), scale, p, seed, offset)
    dx1 = k.softmax_dropout_backward(g4.to(device), x4.to(device), stats1, mask.to(device), scale, p, seed, offset)
    same_up_to_summation_order(out, out1)
    same_up_to_summation_order(stats, stats1)
    same_up_to_summation_order(dx, dx1)
