"""The launch-shape overrides of the softmax, element-wise and Adam kernels
(oslo_tune) change how the work is split over lanes, waves and workgroups,
never the result: every override runs the kernels against the float64 oracle
with the tolerances of the default launch shapes."""
import pytest
import torch

from oslo_amd.torch import _C
from test_gpu_adam import test_multi_tensor_adam_vs_oracle as check_adam
from test_gpu_adam import test_unaligned_views_and_many_tensors as check_adam_views
from test_gpu_eltwise import test_bias_dropout_add as check_bias_dropout_add
from test_gpu_eltwise import test_bias_gelu as check_bias_gelu
from test_gpu_softmax import test_causal as check_causal
from test_gpu_softmax import test_masked as check_masked
from test_gpu_softmax_dropout import test_causal_dropout as check_causal_dropout
from test_gpu_softmax_dropout import test_masked_dropout as check_masked_dropout

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

KEYS = [
    "softmax_rows_per_wave", "softmax_lanes_per_row", "softmax_fwd_elems", "softmax_rows_per_block",
    "eltwise_tile_max", "eltwise_tile_min", "eltwise_unroll", "eltwise_rowgroups", "eltwise_fwd_steps",
    "adam_unroll", "softmax_bias_order", "colsum_defer", "softmax_causal_order", "softmax_bias_group",
    "colsum_slices",
]


@pytest.fixture
def tuned():
    yield
    for key in KEYS:
        _C.tune(key, 0)


SOFTMAX_OVERRIDES = [
    ("softmax_rows_per_wave", 1), ("softmax_rows_per_wave", 2), ("softmax_rows_per_wave", 4),
    ("softmax_lanes_per_row", 1), ("softmax_lanes_per_row", 64),
    ("softmax_fwd_elems", 16), ("softmax_fwd_elems", 32), ("softmax_fwd_elems", 64),
    ("softmax_rows_per_block", 1), ("softmax_rows_per_block", 3), ("softmax_rows_per_block", 4),
    ("softmax_rows_per_block", 16),
    ("softmax_causal_order", 1), ("softmax_causal_order", 2), ("softmax_causal_order", 3),
]

# (sq, sk, dtype): one to eight chunks per lane, one or several waves per row
SOFTMAX_ROWS = [
    (40, 128, BF16), (33, 256, F16), (21, 512, BF16), (19, 512, F32), (17, 768, F16),
    (9, 1024, BF16), (7, 2048, F16), (5, 2048, F32), (5, 4096, BF16), (3, 8192, F16),
]


@pytest.mark.parametrize("key,value", SOFTMAX_OVERRIDES)
@pytest.mark.parametrize("sq,sk,dtype", SOFTMAX_ROWS)
def test_softmax_override_keeps_the_result(device, tuned, sq, sk, dtype, key, value):
    _C.tune(key, value)
    check_causal(device, 2, sq, sk, dtype, 0.25)
    check_masked(device, 2, 2, sq, sk, dtype, 0.25, "padding")
    check_causal_dropout(device, 2, sq, sk, dtype, 0.25, 0.2)
    check_masked_dropout(device, 2, 2, sq, sk, dtype, 0.25, "full", 0.2)


ELTWISE_OVERRIDES = [
    ("eltwise_tile_max", 64), ("eltwise_tile_max", 8), ("eltwise_tile_max", 1),
    ("eltwise_tile_min", 64), ("eltwise_tile_min", 256),
    ("eltwise_unroll", 1), ("eltwise_unroll", 2), ("eltwise_unroll", 4), ("eltwise_unroll", 8),
    ("eltwise_rowgroups", 1), ("eltwise_rowgroups", 7), ("eltwise_rowgroups", 1024),
    ("eltwise_fwd_steps", 2), ("eltwise_fwd_steps", 5),
]

ELTWISE_SHAPES = [
    (517, 64, BF16), (301, 3072, BF16), (67, 11008, F16), (1031, 16, BF16), (129, 96, F32),
    (513, 36, F32), (64, 4096, BF16),
]


@pytest.mark.parametrize("key,value", ELTWISE_OVERRIDES)
@pytest.mark.parametrize("rows,cols,dtype", ELTWISE_SHAPES)
def test_eltwise_override_keeps_the_result(device, tuned, rows, cols, dtype, key, value):
    _C.tune(key, value)
    check_bias_gelu(device, rows, cols, dtype, True)
    check_bias_dropout_add(device, rows, cols, dtype, 0.1, "bias+res")


@pytest.mark.parametrize("unroll", [1, 2, 4])
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_adam_override_keeps_the_result(device, tuned, dtype, unroll):
    _C.tune("adam_unroll", unroll)
    check_adam(device, dtype, 1, 1, 0.01)
    check_adam_views(device)


# ------------------------------------------------------------ bias softmax under the launch overrides
BIAS_OVERRIDES = [
    ("softmax_rows_per_wave", 2), ("softmax_rows_per_wave", 4), ("softmax_lanes_per_row", 1),
    ("softmax_lanes_per_row", 64), ("softmax_fwd_elems", 16), ("softmax_fwd_elems", 64),
    ("softmax_rows_per_block", 3), ("softmax_rows_per_block", 16),
    ("softmax_causal_order", 2), ("softmax_causal_order", 3),
    ("softmax_bias_group", 1), ("softmax_bias_group", 4), ("softmax_bias_group", 256),
]


@pytest.mark.parametrize("key,value", BIAS_OVERRIDES)
@pytest.mark.parametrize("sq,sk,dtype", [(40, 128, BF16), (19, 512, F32), (9, 1024, F16), (5, 4096, BF16),
                                         (7, 2048, F16)])
def test_bias_softmax_override_keeps_the_result(device, tuned, sq, sk, dtype, key, value):
    """The softmax with an additive term under every launch-shape override
    (shapes the defaults never take), with and without the skip of hidden
    chunks and the fused dropout, against the float64 oracle."""
    from test_gpu_softmax_bias import test_bias_softmax as check_bias
    from test_gpu_softmax_bias import test_bias_softmax_dropout as check_bias_dropout

    _C.tune(key, value)
    check_bias(device, 2, 2, sq, sk, dtype, 0.25, "min" if dtype != F16 else "inf", True)
    check_bias(device, 2, 2, sq, sk, dtype, 0.25, "t5", False)
    _C.tune(key, value)  # (check_bias pins and then releases softmax_rows_per_wave)
    check_bias_dropout(device, 2, 2, sq, sk, dtype, 0.25, "perq", False, 0.1)


@pytest.mark.parametrize("order", [1, 2, 3])
@pytest.mark.parametrize("sq,sk,dtype", [(37, 64, F16), (64, 40, BF16), (33, 33, F32), (96, 96, BF16),
                                         (8, 4096, BF16), (5, 2051, BF16), (64, 1024, F16)])
def test_causal_order_with_a_key_mask(device, tuned, sq, sk, dtype, order):
    """Every order of the queries under the diagonal, for the kernels that take
    the diagonal next to a key mask (odd and even numbers of queries, sq != sk)."""
    from test_gpu_softmax_causal_masked import test_causal_masked as check_cm
    from test_gpu_softmax_causal_masked import test_causal_masked_dropout as check_cm_dropout

    _C.tune("softmax_causal_order", order)
    check_cm(device, 2, 2, sq, sk, dtype, 0.25, "right")
    check_cm_dropout(device, 2, 2, sq, sk, dtype, 0.25, "holes", 0.1)


# ------------------------------------------------------------ the column-sum finalize as a call of its own
def test_deferred_finalize_probe_equals_the_entry_point(device, tuned):
    """Measurement hook: with "colsum_defer" the backward entry points stop
    after their main kernel, and oslo_colsum_finalize_probe reduces the partial
    rows they left in the workspace.  The pair gives the bits of the plain call."""
    from helpers import randn

    lib = _C.load_library()
    ln = _C.get_layernorm_kernel()
    n1, n2 = 512, 6144   # one row per step and workgroup: every partial row of the workspace is used
    x = randn((n1, n2), BF16, 1).to(device)
    dy = randn((n1, n2), BF16, 2).to(device)
    gamma = randn((n2,), BF16, 3, std=0.1, mean=1.0).to(device)
    beta = randn((n2,), BF16, 4, std=0.1).to(device)
    _, mean, invvar = ln.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
    dx0, dg0, db0 = ln.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, 1e-5)
    nbytes = int(lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, n1, n2))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    dx, dg, db = torch.empty_like(x), torch.full_like(gamma, float("nan")), torch.full_like(beta, float("nan"))
    st = torch.cuda.current_stream().cuda_stream
    _C.tune("colsum_defer", 1)
    try:
        rc = lib.oslo_ln_bwd(dy.data_ptr(), x.data_ptr(), mean.data_ptr(), invvar.data_ptr(), gamma.data_ptr(),
                             dx.data_ptr(), dg.data_ptr(), db.data_ptr(), ws.data_ptr(), nbytes, n1, n2, 2, 2, st)
        assert rc == 0, lib.oslo_hip_last_error()
    finally:
        _C.tune("colsum_defer", 0)
    torch.cuda.synchronize()
    assert torch.equal(dx, dx0) and torch.isnan(dg.float()).all()   # parameter gradients not written yet
    parts = nbytes // (2 * n2 * 4)
    rc = lib.oslo_colsum_finalize_probe(ws.data_ptr(), parts, n2, dg.data_ptr(), db.data_ptr(), None, 2, st)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    assert torch.equal(dg, dg0) and torch.equal(db, db0)
    assert lib.oslo_colsum_finalize_probe(None, parts, n2, dg.data_ptr(), None, None, 2, st) == -1


@pytest.mark.parametrize("slices", [64, 128, 256])
@pytest.mark.parametrize("parts,cols,dtype", [(256, 6144, BF16), (300, 1024, F32), (7, 36, F16), (1, 4, F32)])
def test_finalize_slices_keep_the_column_sums(device, tuned, parts, cols, dtype, slices):
    """The reduction of the partial rows under every workgroup shape
    ("colsum_slices": 64 or 128 slices of the rows over 32 columns, 256 over
    16 columns), against a float64 sum of the same rows: the shape changes the
    order of the additions, not the addends."""
    lib = _C.load_library()
    g = torch.Generator().manual_seed(parts * 131 + cols)
    part = torch.randn(2, parts, cols, generator=g, dtype=torch.float32)
    want = part.double().sum(dim=1)
    part_d = part.to(device)
    out = torch.full((2, cols), float("nan"), dtype=dtype, device=device)
    st = torch.cuda.current_stream().cuda_stream
    code = {F32: 0, F16: 1, BF16: 2}[dtype]
    _C.tune("colsum_slices", slices)
    rc = lib.oslo_colsum_finalize_probe(part_d.data_ptr(), parts, cols, out[0].data_ptr(), out[1].data_ptr(),
                                        None, code, st)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    # fp32 accumulation of `parts` addends of unit variance, then one rounding to dtype
    scale = float(want.abs().max()) + 1.0
    tol = scale * (parts * 2.0 ** -24 + {F32: 2.0 ** -24, F16: 2.0 ** -11, BF16: 2.0 ** -8}[dtype])
    assert (out.double().cpu() - want).abs().max().item() <= tol
