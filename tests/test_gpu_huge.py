"""Tensors of more than 2^31 elements: every kernel family indexes with 64-bit
offsets.  Inputs are generated on the GPU; rows from the far end of each tensor
(beyond the 32-bit element range) are checked against the oracle."""
import numpy as np
import pytest
import torch

from helpers import check, f64
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C
from test_gpu_fullsize import gpu_randn

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def far_rows(n1, n2):
    """Row indices whose elements start beyond 2^31 and beyond 2^32 where present."""
    rows = {0, n1 - 1, n1 - 2}
    for limit in (2 ** 31, 2 ** 32):
        r = limit // n2 + 1
        if r < n1:
            rows.update((r, min(n1 - 1, r + 7)))
    return torch.tensor(sorted(rows))


def test_norm_and_elementwise_beyond_2_31_elements(device):
    n1, n2 = 140000, 32768  # 4.59e9 elements: beyond 2^32 as well
    assert n1 * n2 > 2 ** 32
    x = gpu_randn((n1, n2), BF16, 1, device)
    gamma = gpu_randn((n2,), BF16, 2, device, std=0.1, mean=1.0)
    beta = gpu_randn((n2,), BF16, 3, device, std=0.1)
    ln = _C.get_layernorm_kernel()
    ek = _C.get_fused_elementwise_kernel()
    rows = far_rows(n1, n2)
    sel = rows.to(device)
    # LayerNorm forward + backward (the backward reuses x as the upstream gradient)
    y, mean, invvar = ln.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
    oy, omean, oinv = cf.layer_norm_fwd(f64(x[sel]), f64(gamma), f64(beta), 1e-5)
    check(y[sel], oy, "huge ln fwd", atol=1e-5)
    assert np.allclose(f64(mean[sel]), omean, atol=1e-5)
    dx, dg, db = ln.layer_norm_backward_affine(y, mean, invvar, x, (n2,), gamma, beta, 1e-5)
    odx, _, _ = cf.layer_norm_bwd(f64(y[sel]), f64(x[sel]), f64(mean[sel]), f64(invvar[sel]), f64(gamma))
    check(dx[sel], odx, "huge ln bwd", atol=1e-5)
    assert torch.isfinite(dg.float()).all() and torch.isfinite(db.float()).all()
    del dx
    # bias-dropout-add forward into y's storage is not allowed (no aliasing): fresh output
    p, seed, offset = 0.1, 11, 4
    out = ek.bias_dropout_add_forward(x, beta, y, p, seed, offset)
    keep = np.stack([philox.keep_mask(n2, p, seed, offset, first_element=int(r) * n2) for r in rows]).astype(bool)
    check(out[sel], cf.bias_dropout_add_fwd(f64(x[sel]), f64(beta), f64(y[sel]), keep, p), "huge bda fwd", atol=1e-6,
          min_exact=0.99)
    del out
    act = ek.bias_gelu_forward(x, beta)
    check(act[sel], cf.bias_gelu_fwd(f64(x[sel]), f64(beta)), "huge gelu fwd", atol=1e-6)
    dact, dbias = ek.bias_gelu_backward(y, x, beta)
    check(dact[sel], cf.bias_gelu_bwd(f64(y[sel]), f64(x[sel]), f64(beta))[0], "huge gelu bwd", atol=1e-6)
    assert torch.isfinite(dbias.float()).all()


def test_softmax_beyond_2_31_elements(device):
    ab, s = 18, 11008  # 2.18e9 elements
    assert ab * s * s > 2 ** 31
    x = gpu_randn((ab, s, s), BF16, 5, device)
    sm = _C.get_softmax_kernel()
    scale, p, seed, offset = 0.125, 0.1, 21, 8
    rows = far_rows(ab * s, s)
    sel = rows.to(device)
    qi = (rows % s).numpy()
    hidden = np.arange(s)[None, :] > qi[:, None]
    y = sm.fused_scaled_upper_triang_masked_softmax_forward(x, scale)
    check(y.view(-1, s)[sel], cf.softmax_masked_fwd(f64(x.view(-1, s)[sel]), hidden, scale), "huge softmax fwd",
          atol=1e-9)
    dx = sm.fused_scaled_upper_triang_masked_softmax_backward(x, y, scale)
    check(dx.view(-1, s)[sel], cf.softmax_bwd(f64(x.view(-1, s)[sel]), f64(y.view(-1, s)[sel]), scale),
          "huge softmax bwd", atol=2e-7)
    del dx, y
    out, stats = sm.softmax_dropout_forward(x, None, scale, p, seed, offset)
    keep = np.stack([philox.keep_mask(s, p, seed, offset, first_element=int(r) * s) for r in rows]).astype(bool)
    check(out.view(-1, s)[sel], cf.softmax_dropout_fwd(f64(x.view(-1, s)[sel]), hidden, scale, keep, p),
          "huge softmax dropout fwd", atol=1e-9)
    ddx = sm.softmax_dropout_backward(out, x, stats, None, scale, p, seed, offset)
    check(ddx.view(-1, s)[sel],
          cf.softmax_dropout_bwd(f64(out.view(-1, s)[sel]), f64(x.view(-1, s)[sel]), hidden, scale, keep, p),
          "huge softmax dropout bwd", atol=3e-7)


def test_softmax_with_more_than_2_31_rows(device):
    """Beyond 2^31 rows the kernels recover (batch, head, query) from the row
    index with 64-bit divisions instead of the 32-bit reciprocal multiply:
    short rows (8 keys), 2.15e9 of them, rows on both sides of 2^31 checked."""
    sk = 8
    sm = _C.get_softmax_kernel()
    # causal [attn_batches, sq, sk], sq = sk
    ab = 4097 * 65536  # = 4097 * 64 * 8192 / 8: the same tensor serves the [b, heads, sq, sk] case below
    rows_total = ab * sk
    assert rows_total > 2 ** 31
    x = gpu_randn((ab, sk, sk), BF16, 9, device, std=2.0)
    y = sm.fused_scaled_upper_triang_masked_softmax_forward(x, 0.5)
    rows = torch.tensor(sorted({0, 1, 7, 8, 2 ** 31 - 9, 2 ** 31 - 1, 2 ** 31, 2 ** 31 + 1, 2 ** 31 + 11,
                                rows_total - 9, rows_total - 2, rows_total - 1}))
    sel = rows.to(device)
    qi = (rows % sk).numpy()
    hidden = np.arange(sk)[None, :] > qi[:, None]
    check(y.view(-1, sk)[sel], cf.softmax_masked_fwd(f64(x.view(-1, sk)[sel]), hidden, 0.5), "causal fwd", atol=1e-9)
    # whole-tensor property on a slab around 2^31: the zeros sit above the diagonal, rows sum to 1
    b0 = 2 ** 28 - 4096
    slab = y[b0:b0 + 8192].float()
    assert torch.triu(slab, diagonal=1).count_nonzero().item() == 0
    assert (slab.sum(-1) - 1).abs().max().item() <= 1e-2
    assert (slab[:, 0, 0] == 1).all()
    del y, slab
    # key padding [b, np, sq, sk] with one mask row per batch entry: b and np both matter
    b, heads, sq = 4097, 64, 8192
    assert b * heads * sq == x.numel() // sk
    x4 = x.view(b, heads, sq, sk)
    valid = torch.randint(1, sk + 1, (b,), generator=torch.Generator().manual_seed(3))
    pad = torch.arange(sk)[None, :] >= valid[:, None]
    y4 = sm.fused_scaled_masked_softmax_forward(x4, pad.view(b, 1, 1, sk).to(device), 0.5)
    bi = (rows // (heads * sq)).numpy()
    hidden = pad.numpy()[bi]
    check(y4.view(-1, sk)[sel], cf.softmax_masked_fwd(f64(x.view(-1, sk)[sel]), hidden, 0.5), "padding fwd", atol=1e-9)
    # every batch entry: exactly its padded keys are zero (a wrong batch index would show at some entry)
    for e in (0, 1, 2047, 2048, 2049, 4095, 4096):
        ye = y4[e, ::16, ::512].float()
        v = int(valid[e])
        assert ye[..., v:].count_nonzero().item() == 0
        assert (ye[..., :v] > 0).all()
    # the backward and the dropout pair at this row count (x doubles as the incoming gradient)
    hidden = np.arange(sk)[None, :] > qi[:, None]
    y = y4.view(ab, sk, sk)
    del y4
    y = sm.fused_scaled_upper_triang_masked_softmax_forward(x, 0.5)
    dx = sm.fused_scaled_upper_triang_masked_softmax_backward(x, y, 0.5)
    check(dx.view(-1, sk)[sel], cf.softmax_bwd(f64(x.view(-1, sk)[sel]), f64(y.view(-1, sk)[sel]), 0.5),
          "causal bwd", atol=2e-7)
    del dx, y
    p, seed, offset = 0.2, 5, 16
    out, stats = sm.softmax_dropout_forward(x, None, 0.5, p, seed, offset)
    keep = np.stack([philox.keep_mask(sk, p, seed, offset, first_element=int(r) * sk) for r in rows]).astype(bool)
    check(out.view(-1, sk)[sel], cf.softmax_dropout_fwd(f64(x.view(-1, sk)[sel]), hidden, 0.5, keep, p),
          "causal dropout fwd", atol=1e-9)
    ddx = sm.softmax_dropout_backward(out, x, stats, None, 0.5, p, seed, offset)
    check(ddx.view(-1, sk)[sel],
          cf.softmax_dropout_bwd(f64(out.view(-1, sk)[sel]), f64(x.view(-1, sk)[sel]), hidden, 0.5, keep, p),
          "causal dropout bwd", atol=3e-7, min_exact=0.98)


def test_elementwise_forward_beyond_2_32_work_items(device):
    """A dispatch holds fewer than 2^32 work-items: a forward with one 128-bit
    vector per lane over 1.72e10 fp32 elements takes two launches.  Rows on both
    sides of the split, and the last ones, against the oracle."""
    n2 = 1024
    n1 = (2 ** 32 // 256) * 256 * 4 // n2 + 4096  # just beyond 2^32 lanes of 4 elements
    assert n1 * n2 // 4 > 2 ** 32
    F32 = torch.float32
    x = gpu_randn((n1, n2), F32, 13, device)
    bias = gpu_randn((n2,), F32, 14, device, std=0.1)
    k = _C.get_fused_elementwise_kernel()
    _C.tune("eltwise_unroll", 1)
    try:
        y = k.bias_gelu_forward(x, bias)
    finally:
        _C.tune("eltwise_unroll", 0)
    split = 2 ** 32 * 4 // n2  # first row of the second launch
    rows = torch.tensor(sorted({0, 1, split - 2, split - 1, split, split + 1, n1 - 2, n1 - 1}))
    sel = rows.to(device)
    check(y[sel], cf.bias_gelu_fwd(f64(x[sel]), f64(bias)), "huge bias-GeLU fwd", atol=1e-7)
    assert torch.isfinite(y[-8192:]).all() and y[-8192:].abs().sum().item() > 0


def test_norm_with_more_than_2_31_rows(device):
    """LayerNorm and RMSNorm over 2.15e9 rows of 8 elements: row indices beyond 32 bits in the
    side-by-side short-row kernels, forward and backward, rows on both sides of 2^31."""
    n2 = 8
    n1 = 2 ** 31 + 4104
    x = gpu_randn((n1, n2), BF16, 21, device, std=1.5, mean=0.25)
    gamma = gpu_randn((n2,), BF16, 22, device, std=0.1, mean=1.0)
    beta = gpu_randn((n2,), BF16, 23, device, std=0.1)
    k = _C.get_layernorm_kernel()
    rows = torch.tensor(sorted({0, 1, 63, 64, 2 ** 31 - 65, 2 ** 31 - 1, 2 ** 31, 2 ** 31 + 1, 2 ** 31 + 77,
                                n1 - 65, n1 - 2, n1 - 1}))
    sel = rows.to(device)
    y, mean, invvar = k.layer_norm_forward_affine(x, (n2,), gamma, beta, 1e-5)
    oy, omean, oinv = cf.layer_norm_fwd(f64(x[sel]), f64(gamma), f64(beta), 1e-5, "bf16")
    check(y[sel], oy, "huge-n1 ln fwd", atol=2e-5, max_ulp=2, min_exact=0.97)
    assert np.allclose(f64(mean[sel]), omean, rtol=1e-5, atol=1e-6)
    assert np.allclose(f64(invvar[sel]), oinv, rtol=1e-5)
    # x doubles as the incoming gradient
    dx, dg, db = k.layer_norm_backward_affine(x, mean, invvar, x, (n2,), gamma, beta, 1e-5)
    odx, _, _ = cf.layer_norm_bwd(f64(x[sel]), f64(x[sel]), f64(mean[sel]), f64(invvar[sel]), f64(gamma))
    amp = float(np.abs(f64(invvar[sel])).max()) * 8.0
    check(dx[sel], odx, "huge-n1 ln dx", atol=2e-5 + 2.5e-7 * amp)
    # dbeta = column sums of dy over all 2.15e9 rows (float64 on the GPU, in slabs)
    want_db = torch.zeros(n2, dtype=torch.float64, device=device)
    for r0 in range(0, n1, 2 ** 27):
        want_db += x[r0:r0 + 2 ** 27].double().sum(0)
    assert torch.allclose(db.double(), want_db, rtol=2e-2, atol=50.0), (db, want_db)
    del y, dx
    y, invvar = k.rms_norm_forward_affine(x, (n2,), gamma, 1e-5)
    oy, _ = cf.rms_norm_fwd(f64(x[sel]), f64(gamma), 1e-5, "bf16")
    check(y[sel], oy, "huge-n1 rms fwd", atol=2e-5, max_ulp=2, min_exact=0.97)


def test_elementwise_with_more_than_2_31_rows(device):
    """bias-GeLU and bias-dropout-add over 2.15e9 rows of 8 columns, forward and backward."""
    n2 = 8
    n1 = 2 ** 31 + 4104
    x = gpu_randn((n1, n2), BF16, 31, device)
    bias = gpu_randn((n2,), BF16, 32, device, std=0.1)
    ek = _C.get_fused_elementwise_kernel()
    rows = torch.tensor(sorted({0, 1, 255, 256, 2 ** 31 - 257, 2 ** 31 - 1, 2 ** 31, 2 ** 31 + 1, 2 ** 31 + 300,
                                n1 - 257, n1 - 2, n1 - 1}))
    sel = rows.to(device)
    act = ek.bias_gelu_forward(x, bias)
    check(act[sel], cf.bias_gelu_fwd(f64(x[sel]), f64(bias)), "huge-n1 gelu fwd", atol=1e-6)
    dact, dbias = ek.bias_gelu_backward(act, x, bias)
    check(dact[sel], cf.bias_gelu_bwd(f64(act[sel]), f64(x[sel]), f64(bias))[0], "huge-n1 gelu bwd", atol=1e-6)
    want = torch.zeros(n2, dtype=torch.float64, device=device)
    for r0 in range(0, n1, 2 ** 27):
        want += dact[r0:r0 + 2 ** 27].double().sum(0)
    assert torch.allclose(dbias.double(), want, rtol=2e-2, atol=50.0), (dbias, want)
    del dact
    p, seed, offset = 0.1, 11, 4
    out = ek.bias_dropout_add_forward(x, bias, act, p, seed, offset)
    keep = np.stack([philox.keep_mask(n2, p, seed, offset, first_element=int(r) * n2) for r in rows]).astype(bool)
    check(out[sel], cf.bias_dropout_add_fwd(f64(x[sel]), f64(bias), f64(act[sel]), keep, p), "huge-n1 bda fwd",
          atol=1e-6, min_exact=0.97)
    del out, act
    dx, db = ek.bias_dropout_add_backward(x, p, seed, offset)
    want_dx = np.where(keep, f64(x[sel]) / (1.0 - p), 0.0)
    check(dx[sel], want_dx, "huge-n1 bda bwd", atol=1e-6, min_exact=0.97)


def test_adam_on_a_tensor_beyond_2_31_elements(device):
    n = 2 ** 31 + 4099
    g = torch.empty(n, device=device, dtype=BF16).normal_()
    p = torch.empty(n, device=device, dtype=BF16).normal_()
    m = torch.zeros(n, device=device, dtype=BF16)
    v = torch.zeros(n, device=device, dtype=BF16)
    tail = slice(n - 5000, n)
    head = slice(0, 5000)
    p0 = [f64(p[head]), f64(p[tail])]
    g0 = [f64(g[head]), f64(g[tail])]
    _C.get_adam_kernel().multi_tensor_adam(0, None, [[g], [p], [m], [v]], 1e-2, 0.9, 0.999, 1e-8, 1, 1, 1, 0.01)
    for sl, pp, gg in ((head, p0[0], g0[0]), (tail, p0[1], g0[1])):
        want = cf.adam_step(gg, pp, np.zeros_like(pp), np.zeros_like(pp), 1e-2, 0.9, 0.999, 1e-8, 1, 1, True, 0.01)
        check(p[sl], want[0], "huge adam p", atol=5e-7, min_exact=0.99)
        check(m[sl], want[1], "huge adam m", atol=1e-7, min_exact=0.99)
        check(v[sl], want[2], "huge adam v", atol=1e-8, min_exact=0.99)


def test_optimizer_family_on_a_tensor_beyond_2_31_elements(device):
    """The generic multi-tensor kernel (here: SGD with momentum, next to a short
    tensor in the same launch) and the norm kernels index with 64-bit offsets."""
    n = 2 ** 31 + 4099
    g = torch.empty(n, device=device, dtype=BF16).normal_()
    w = torch.empty(n, device=device, dtype=BF16).normal_()
    mom = torch.empty(n, device=device, dtype=BF16).normal_()
    small = [torch.ones(100, device=device, dtype=BF16) for _ in range(3)]
    tail, head = slice(n - 5000, n), slice(0, 5000)
    before = [(f64(g[s]), f64(w[s]), f64(mom[s])) for s in (head, tail)]
    # the norm first (it reads the gradients the step leaves alone): against torch in float64 on slices
    total, per = _C.get_l2norm_kernel().multi_tensor_l2norm(0, None, [[g, small[0]]], True)
    sumsq = sum(float(g[i:i + (1 << 28)].double().square().sum()) for i in range(0, n, 1 << 28))
    assert np.isclose(per[0].item(), np.sqrt(sumsq), rtol=1e-5) and np.isclose(per[1].item(), 10.0, rtol=1e-6)
    assert np.isclose(total.item(), np.sqrt(sumsq + 100.0), rtol=1e-5)
    _C.get_sgd_kernel().multi_tensor_sgd(0, None, [[g, small[0]], [w, small[1]], [mom, small[2]]],
                                         0.01, 0.9, 0.0, 0.05, False, False, False, 1.0)
    for s, (gg, ww, mm) in zip((head, tail), before):
        want_w, want_m, _ = cf.sgd_step(gg, ww, mm, 0.05, 0.01, 0.9, 0.0, False, False)
        check(w[s], want_w, "huge sgd w", atol=1e-6, min_exact=0.95, single_rounding_too=True)
        check(mom[s], want_m, "huge sgd momentum", atol=1e-6, min_exact=0.95, single_rounding_too=True)
    # g = w = mom = 1: mom' = 0.9 + (1 + 0.01) = 1.91, w' = 1 - 0.05 * 1.91
    assert torch.equal(small[2], torch.full_like(small[2], 1.91)) and torch.equal(small[1], torch.full_like(small[1], 0.9045))
