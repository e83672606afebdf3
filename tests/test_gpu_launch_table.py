"""Every build of the register kernels behind a launch table is a parity
obligation of its own: the launch code picks a build from the row length, the
dtypes and the launch overrides (oslo_tune), and a build that no test reaches
could differ from its siblings unnoticed.  These sweeps walk the tables: row
lengths chosen by the number of 16-byte chunks they hold (so that every lane
group width, chunk count per lane, even / ragged tail and workgroup size
comes up for every dtype), under the defaults and under the overrides that
select another build, each against the float64 oracle through the checks of
the per-op test files.  An override that a shape has no build for is refused
by the library (RuntimeError) and skipped.

The full sweep (2200 runs of a shape under a setting, four minutes) runs with
OSLO_LAUNCH_TABLE=full.  By default each shape runs only the settings that
golden/launch_table_cover.json lists for it: a smallest set of (shape, setting)
pairs that between them launch every kernel build the full sweep launches,
taken from a kernel trace of the full sweep (rocprofv3 --kernel-trace, the
runs told apart by marker launches) by golden/make_launch_table_cover.py.
After a change of a launch rule the table is made again from such a trace."""
import json
import os

import pytest
import torch

from helpers import randn
from oslo_amd.torch import _C
from test_gpu_eltwise import test_bias_dropout_add as check_bda
from test_gpu_eltwise import test_bias_gelu as check_gelu
from test_gpu_norm import test_layer_norm as check_layer_norm
from test_gpu_norm import test_rms_norm as check_rms_norm
from test_gpu_residual_norm import test_fused_vs_oracle as check_fused
from test_gpu_softmax import test_causal as check_causal
from test_gpu_softmax import test_masked as check_masked
from test_gpu_softmax_bias import test_bias_softmax as check_bias
from test_gpu_softmax_bias import test_bias_softmax_dropout as check_bias_dropout
from test_gpu_softmax_dropout import test_causal_dropout as check_causal_dropout
from test_gpu_softmax_dropout import test_masked_dropout as check_masked_dropout

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

KEYS = [
    "softmax_rows_per_wave", "softmax_lanes_per_row", "softmax_fwd_elems", "softmax_rows_per_block",
    "norm_fwd_vpl", "norm_fwd_waves", "norm_fwd_iters", "norm_bwd_vpl", "norm_bwd_prefetch",
    "norm_bwd_waves", "norm_bwd_blocks_per_cu", "norm_lanes_per_row",
    "eltwise_unroll", "eltwise_tile_max", "eltwise_tile_min", "eltwise_fwd_steps",
]


@pytest.fixture
def tuned():
    yield
    for key in KEYS:
        _C.tune(key, 0)


def _chunk(dtype):
    return 4 if dtype == F32 else 8


FULL = os.environ.get("OSLO_LAUNCH_TABLE", "") == "full"
with open(os.path.join(os.path.dirname(__file__), "golden", "launch_table_cover.json")) as _f:
    COVER = json.load(_f)


DTYPE = {"f32": F32, "f16": F16, "bf16": BF16}


def _shapes(family, names, sizes):
    """(dtype name, size) pairs of a sweep: all of them in the full sweep,
    else the ones the cover table has settings for."""
    return [(n, c) for n in names for c in sizes if FULL or "%s:%d" % (n, c) in COVER[family]]


def _settings(family, name, size, full_settings):
    """The settings a shape runs under: the defaults and all of them in the
    full sweep, else the ones the cover table lists."""
    if FULL:
        return [{}] + list(full_settings)
    return COVER[family]["%s:%d" % (name, size)]


# ------------------------------------------------------------------ softmax
# chunks per row: lane groups of 8 / 16 / 32, their two- and three-chunk
# forms, one to eight chunks per lane of a whole wave, several waves per row
# (a ragged tail is no build of its own in these kernels: three ragged lengths)
SOFTMAX_CHUNKS = [5, 8, 12, 16, 20, 24, 32, 48, 50, 64, 96, 128, 192, 256, 300, 512, 1024, 2048]


def _softmax_settings(chunks):
    s = []
    if chunks <= 256:
        s += [{"softmax_rows_per_wave": v} for v in (1, 2, 4)]
    if chunks <= 192:
        s += [{"softmax_lanes_per_row": 64}, {"softmax_lanes_per_row": 1},
              {"softmax_lanes_per_row": 64, "softmax_rows_per_wave": 2},
              {"softmax_lanes_per_row": 64, "softmax_rows_per_wave": 4}]
    if chunks <= 16:
        s += [{"softmax_lanes_per_row": 32}, {"softmax_lanes_per_row": 32, "softmax_rows_per_wave": 1}]
    if chunks <= 8:
        s += [{"softmax_lanes_per_row": 16}, {"softmax_lanes_per_row": 16, "softmax_rows_per_wave": 2}]
    if chunks >= 64:
        s += [{"softmax_fwd_elems": 16}, {"softmax_fwd_elems": 64},
              {"softmax_fwd_elems": 64, "softmax_rows_per_wave": 2},
              {"softmax_fwd_elems": 64, "softmax_rows_per_wave": 4}]
    return s


def _softmax_checks(device, dtype, sq, sk, setting):
    # (the masked kernels take the diagonal as a run-time flag: no build of its own)
    rpw = setting.get("softmax_rows_per_wave", 0)
    check_causal(device, 2, sq, sk, dtype, 0.25)
    check_causal_dropout(device, 2, sq, sk, dtype, 0.25, 0.1)
    check_masked(device, 2, 1, sq, sk, dtype, 0.25, "padding")
    check_masked_dropout(device, 2, 1, sq, sk, dtype, 0.25, "padding", 0.1)
    check_bias(device, 2, 2, sq, sk, dtype, 0.25, "t5", False, rows_per_wave=(rpw, rpw) if setting else (1, 0))
    check_bias_dropout(device, 2, 2, sq, sk, dtype, 0.25, "perq", True, 0.1)


def _under_each(settings, run):
    """Runs `run(setting)` under each setting (a dict of overrides, empty for
    the defaults); returns how many settings the library had a build for."""
    done = 0
    for setting in settings:
        for key in KEYS:
            _C.tune(key, 0)
        for key, value in setting.items():
            _C.tune(key, value)
        try:
            run(setting)
        except RuntimeError as e:
            # a refused override: no build of the kernel for this shape
            if not setting or not any(s in str(e) for s in ("no kernel", "needs a workgroup", "built for")):
                raise
            continue
        done += 1
    return done


@pytest.mark.parametrize("name,chunks", _shapes("softmax", ["f32", "f16", "bf16"], SOFTMAX_CHUNKS))
def test_softmax_launch_table(device, tuned, name, chunks):
    dtype = DTYPE[name]
    sk = chunks * _chunk(dtype)
    settings = _settings("softmax", name, chunks, _softmax_settings(chunks))
    assert _under_each(settings, lambda s: _softmax_checks(device, dtype, 5, sk, s)) >= 1


def test_softmax_fp32_rows_of_eight_chunks_per_lane(device, tuned):
    """fp32 rows beyond 16384 keys: the backward passes hold eight chunks per lane."""
    _softmax_checks(device, F32, 3, 8192 * 4, {})
    _softmax_checks(device, F32, 3, 5000 * 4, {})


# lengths that are no multiple of the 16-byte chunk: one wave per row with
# 8-, 4- or 2-byte accesses (fp32: 8 or 4) in builds for rows of up to 256,
# 1024 and 2048 keys, and one workgroup per row beyond
@pytest.mark.parametrize("sk", [50, 51, 100, 514, 515, 516, 1538, 1539, 1540, 2051, 2054])
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_softmax_rows_off_the_chunk_grid(device, tuned, dtype, sk):
    _softmax_checks(device, dtype, 5, sk, {})


# ------------------------------------------------------------------ norms
NORM_CHUNKS = [5, 8, 12, 16, 20, 24, 32, 48, 50, 64, 96, 100, 128, 192, 200, 256, 300, 384, 512, 640, 768,
               1000, 1024, 1536, 2048, 3000, 4096]

NORM_SETTINGS = [
    {"norm_fwd_vpl": 1, "norm_bwd_vpl": 1, "norm_bwd_prefetch": 1},
    {"norm_fwd_vpl": 2, "norm_bwd_vpl": 2, "norm_bwd_prefetch": 2},
    {"norm_fwd_vpl": 3, "norm_bwd_vpl": 4, "norm_bwd_prefetch": 1},
    {"norm_fwd_vpl": 4, "norm_bwd_vpl": 4, "norm_bwd_prefetch": 2},
    {"norm_fwd_vpl": 8, "norm_bwd_vpl": 2, "norm_bwd_prefetch": 1, "norm_bwd_waves": 16},
    {"norm_fwd_waves": 16, "norm_bwd_waves": 4, "norm_bwd_prefetch": 2},
    {"norm_fwd_waves": 1, "norm_bwd_waves": 8, "norm_bwd_vpl": 1, "norm_bwd_prefetch": 2},
    {"norm_fwd_waves": 8, "norm_fwd_vpl": 2, "norm_bwd_waves": 12, "norm_bwd_vpl": 2},
    {"norm_fwd_waves": 16, "norm_fwd_vpl": 1, "norm_bwd_waves": 16, "norm_bwd_vpl": 1, "norm_bwd_prefetch": 1},
    {"norm_bwd_waves": 12, "norm_bwd_vpl": 2, "norm_bwd_prefetch": 2},
]
NORM_SHORT_SETTINGS = [{"norm_lanes_per_row": 64}, {"norm_lanes_per_row": 32}, {"norm_lanes_per_row": 16}]


@pytest.mark.parametrize("name,chunks", _shapes("norm", ["f32-f32", "f16-f16", "bf16-bf16", "f32-f16", "f32-bf16"],
                                                 NORM_CHUNKS))
def test_norm_launch_table(device, tuned, name, chunks):
    tin, tout = (DTYPE[n] for n in name.split("-"))   # input dtype, dtype of the parameters and the output
    n2 = chunks * _chunk(tin)
    n1 = 11 if n2 <= 4096 else 5

    def run():
        check_layer_norm(device, n1, n2, tin, tout, True)
        check_rms_norm(device, n1, n2, tin, tout, True)
        if tin == tout:
            check_fused(device, n1, n2, tin, 0.1, False)
            check_fused(device, n1, n2, tin, 0.1, True)

    settings = _settings("norm", name, chunks, NORM_SETTINGS + (NORM_SHORT_SETTINGS if chunks <= 96 else []))
    assert _under_each(settings, lambda s: run()) >= 1


# ------------------------------------------------------------------ element-wise kernels
ELTWISE_SETTINGS = [{"eltwise_unroll": v} for v in (1, 2, 4, 8)] + [
    {"eltwise_fwd_steps": 4}, {"eltwise_tile_max": 256}, {"eltwise_tile_min": 64},
]


@pytest.mark.parametrize("name,cols", _shapes("eltwise", ["f32", "f16", "bf16"], [40, 768, 4096]))
def test_elementwise_launch_table(device, tuned, name, cols):
    dtype = DTYPE[name]
    rows = 37

    def run():
        check_gelu(device, rows, cols, dtype, True)
        check_gelu(device, rows, cols, dtype, False)
        for parts in ("bias+res", "bias", "res", "none"):
            check_bda(device, rows, cols, dtype, 0.1, parts)
            check_bda(device, rows, cols, dtype, 0.0, parts)

    settings = _settings("eltwise", name, cols, ELTWISE_SETTINGS)
    assert _under_each(settings, lambda s: run()) >= 1


# ------------------------------------------------------------------ column sums without a workspace
def _close(a, b, dtype):
    scale = b.float().abs().max().item() + 1e-6
    tol = {F32: 2e-5, F16: 2e-3, BF16: 1.6e-2}[dtype] * scale
    assert (a.float() - b.float()).abs().max().item() <= tol


@pytest.mark.parametrize("tin,tout", [(F32, F32), (F16, F16), (BF16, BF16), (F32, F16), (F32, BF16)])
def test_norm_backward_off_the_chunk_grid_without_a_workspace(device, tin, tout):
    """A caller of the C ABI may pass no workspace where the row length is off
    the 16-byte grid: the parameter gradients then come from one thread per
    column.  Same values as with the workspace the binding brings, up to the
    order of the fp32 additions."""
    lib = _C.load_library()
    ln = _C.get_layernorm_kernel()
    code = {F32: 0, F16: 1, BF16: 2}
    n1, n2 = 45, 33
    x = randn((n1, n2), tin, 1).to(device)
    dy = randn((n1, n2), tout, 2).to(device)
    gamma = randn((n2,), tout, 3, std=0.1, mean=1.0).to(device)
    beta = randn((n2,), tout, 4, std=0.1).to(device)
    st = torch.cuda.current_stream().cuda_stream
    mixed = tin != tout
    fwd = ln.layer_norm_forward_affine_mixed_dtypes if mixed else ln.layer_norm_forward_affine
    _, mean, invvar = fwd(x, (n2,), gamma, beta, 1e-5)
    dx0, dg0, db0 = ln.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, 1e-5)
    dx, dg, db = torch.empty_like(x), torch.empty_like(gamma), torch.empty_like(beta)
    rc = lib.oslo_ln_bwd(dy.data_ptr(), x.data_ptr(), mean.data_ptr(), invvar.data_ptr(), gamma.data_ptr(),
                         dx.data_ptr(), dg.data_ptr(), db.data_ptr(), None, 0, n1, n2, code[tin], code[tout], st)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    assert torch.equal(dx, dx0)
    _close(dg, dg0, tout)
    _close(db, db0, tout)
    rfwd = ln.rms_norm_forward_affine_mixed_dtypes if mixed else ln.rms_norm_forward_affine
    _, rinv = rfwd(x, (n2,), gamma, 1e-5)
    rdx0, rdg0 = ln.rms_norm_backward_affine(dy, rinv, x, (n2,), gamma, 1e-5)
    rdx, rdg = torch.empty_like(x), torch.empty_like(gamma)
    rc = lib.oslo_rms_bwd(dy.data_ptr(), x.data_ptr(), rinv.data_ptr(), gamma.data_ptr(), rdx.data_ptr(),
                          rdg.data_ptr(), None, 0, n1, n2, code[tin], code[tout], st)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    assert torch.equal(rdx, rdx0)
    _close(rdg, rdg0, tout)


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_bias_gradients_off_the_chunk_grid_without_a_workspace(device, dtype):
    """The same for the bias gradients of bias-GeLU, bias-dropout-add and the
    bias-dropout-add inside a norm."""
    lib = _C.load_library()
    el = _C.get_fused_elementwise_kernel()
    ln = _C.get_layernorm_kernel()
    code = {F32: 0, F16: 1, BF16: 2}[dtype]
    rows, cols = 45, 33
    st = torch.cuda.current_stream().cuda_stream
    x = randn((rows, cols), dtype, 1).to(device)
    g = randn((rows, cols), dtype, 2).to(device)
    bias = randn((cols,), dtype, 3, std=0.1).to(device)
    # bias-GeLU
    dx0, db0 = el.bias_gelu_backward(g, x, bias)
    dx, db = torch.empty_like(x), torch.empty_like(bias)
    rc = lib.oslo_bias_gelu_bwd(g.data_ptr(), x.data_ptr(), bias.data_ptr(), dx.data_ptr(), db.data_ptr(),
                                None, 0, rows, cols, code, st)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    assert torch.equal(dx, dx0)
    _close(db, db0, dtype)
    # bias-dropout-add, with and without the input gradient
    p, seed, offset = 0.1, 77, 16
    dx0, db0 = el.bias_dropout_add_backward(g, p, seed, offset)
    for want_dx in (True, False):
        dx, db = torch.empty_like(x), torch.empty_like(bias)
        rc = lib.oslo_bias_dropout_add_bwd(g.data_ptr(), dx.data_ptr() if want_dx else None, db.data_ptr(),
                                           None, 0, rows, cols, p, seed, offset, code, st)
        assert rc == 0, lib.oslo_hip_last_error()
        torch.cuda.synchronize()
        assert not want_dx or torch.equal(dx, dx0)
        _close(db, db0, dtype)
    # bias-dropout-add inside LayerNorm
    res = randn((rows, cols), dtype, 4).to(device)
    gamma = randn((cols,), dtype, 5, std=0.1, mean=1.0).to(device)
    beta = randn((cols,), dtype, 6, std=0.1).to(device)
    dh = randn((rows, cols), dtype, 7).to(device)
    _, h, mean, invvar = ln.bias_dropout_add_norm_forward(False, x, bias, res, (cols,), gamma, beta, 1e-5, p,
                                                          seed, offset)
    r0 = ln.bias_dropout_add_norm_backward(False, g, dh, h, mean, invvar, (cols,), gamma, p, seed, offset)
    dres, dxd = torch.empty_like(x), torch.empty_like(x)
    dg, dbt, dbias = torch.empty_like(gamma), torch.empty_like(beta), torch.empty_like(bias)
    rc = lib.oslo_bias_dropout_add_norm_bwd(g.data_ptr(), dh.data_ptr(), h.data_ptr(), mean.data_ptr(),
                                            invvar.data_ptr(), gamma.data_ptr(), dres.data_ptr(), dxd.data_ptr(),
                                            dg.data_ptr(), dbt.data_ptr(), dbias.data_ptr(), None, 0, rows, cols,
                                            p, seed, offset, 0, code, st)
    assert rc == 0, lib.oslo_hip_last_error()
    torch.cuda.synchronize()
    assert torch.equal(dres, r0[0]) and torch.equal(dxd, r0[1])
    _close(dg, r0[2], dtype)
    _close(dbt, r0[3], dtype)
    _close(dbias, r0[4], dtype)
