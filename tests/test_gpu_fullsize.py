"""The five BASELINE.json workloads at full size on the GPU, through the C ABI.

The float64 oracle would take minutes on tensors of up to 10^9 elements, so each
workload is checked (a) on a sample of whole rows against the oracle, with the
tolerances of tests/helpers.py, and (b) over the entire tensor through
size-independent properties: softmax rows sum to 1 and hidden keys are exact
zeros, gradients of a softmax row sum to 0, column gradients equal the column
sums of what was stored, dropout masks equal the Philox oracle on windows, and
p = 0 is bit-exact.
"""
import math

import numpy as np
import pytest
import torch

from helpers import check, f64
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16


def gpu_randn(shape, dtype, seed, device, std=1.0, mean=0.0):
    g = torch.Generator(device=device).manual_seed(seed)
    out = torch.empty(shape, dtype=dtype, device=device)
    # generate in slabs to bound the fp32 temporary
    flat = out.view(-1)
    step = 1 << 28
    for s in range(0, flat.numel(), step):
        e = min(s + step, flat.numel())
        flat[s:e] = (torch.randn(e - s, generator=g, device=device) * std + mean).to(dtype)
    return out


def sample_rows(nrows, k=48, seed=0):
    r = np.random.default_rng(seed)
    idx = {0, 1, nrows // 2, nrows - 2, nrows - 1}
    idx.update(int(i) for i in r.integers(0, nrows, size=k))
    return torch.tensor(sorted(idx))


# --------------------------------------------------------------------------- cfg1 / cfg5
@pytest.mark.parametrize(
    "name,ab,s,dtype,scale",
    [("cfg1", 48, 512, F32, 0.125), ("cfg5", 256, 2048, BF16, 1.0 / math.sqrt(96.0))],
)
def test_causal_softmax_full_size(device, name, ab, s, dtype, scale):
    x = gpu_randn((ab, s, s), dtype, 1, device)
    g = gpu_randn((ab, s, s), dtype, 2, device)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x, scale)
    dx = k.fused_scaled_upper_triang_masked_softmax_backward(g, y, scale)
    # (b) whole-tensor properties
    tol = 1e-5 if dtype == F32 else 2e-3
    for b0 in range(0, ab, 32):
        yb = y[b0:b0 + 32].float()
        assert (yb.sum(-1) - 1).abs().max().item() <= tol
        assert torch.triu(yb, diagonal=1).count_nonzero().item() == 0
        assert (yb[:, 0, 0] == 1).all()
        assert ((yb > 0).sum(-1) <= torch.arange(1, s + 1, device=device)).all()
        dxb = dx[b0:b0 + 32].float()
        assert torch.triu(dxb, diagonal=1).count_nonzero().item() == 0
        gscale = g[b0:b0 + 32].float().abs().amax(-1) * abs(scale)
        assert (dxb.sum(-1).abs() <= (4 * tol) * gscale + 1e-6).all()
    # (a) sampled rows against the oracle
    rows = sample_rows(ab * s)
    xb = x.view(ab * s, s)[rows.to(device)].cpu()
    yb = y.view(ab * s, s)[rows.to(device)].cpu()
    gb = g.view(ab * s, s)[rows.to(device)].cpu()
    dxb = dx.view(ab * s, s)[rows.to(device)].cpu()
    qi = (rows % s).numpy()
    hidden = np.arange(s)[None, :] > qi[:, None]
    check(yb, cf.softmax_masked_fwd(f64(xb), hidden, scale), name + " fwd rows", atol=1e-9)
    check(dxb, cf.softmax_bwd(f64(gb), f64(yb), scale), name + " bwd rows", atol=1e-7)


@pytest.mark.parametrize(
    "name,ab,s,dtype,scale",
    [("cfg1", 48, 512, F32, 0.125), ("cfg5", 256, 2048, BF16, 1.0 / math.sqrt(96.0))],
)
def test_causal_softmax_dropout_full_size(device, name, ab, s, dtype, scale):
    """Softmax with fused dropout at full size: the keep decisions equal the
    Philox mask of the flattened output, kept values are the plain
    probabilities over 1 - p, gradient rows sum to 0, sampled rows match the
    oracle."""
    p, seed, offset = 0.1, 4242, 16
    x = gpu_randn((ab, s, s), dtype, 1, device)
    g = gpu_randn((ab, s, s), dtype, 2, device)
    k = _C.get_softmax_kernel()
    ek = _C.get_fused_elementwise_kernel()
    out, stats = k.softmax_dropout_forward(x, None, scale, p, seed, offset)
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x, scale)
    keep = ek.philox_mask(x.numel(), p, seed, offset, device).view(ab, s, s)
    tol = 1e-5 if dtype == F32 else 2.0 ** -7
    for b0 in range(0, ab, 32):
        ob, yb, kb = out[b0:b0 + 32].float(), y[b0:b0 + 32].float(), keep[b0:b0 + 32].bool()
        assert ob[~kb].count_nonzero().item() == 0
        assert torch.triu(ob, diagonal=1).count_nonzero().item() == 0
        want = yb / (1.0 - p)
        assert ((ob - want)[kb].abs() <= tol * want[kb] + 1e-30).all()
    del y, keep
    dx = k.softmax_dropout_backward(g, x, stats, None, scale, p, seed, offset)
    for b0 in range(0, ab, 32):
        dxb = dx[b0:b0 + 32].float()
        assert torch.triu(dxb, diagonal=1).count_nonzero().item() == 0
        gscale = g[b0:b0 + 32].float().abs().amax(-1) * abs(scale) / (1.0 - p)
        rtol = 1e-5 if dtype == F32 else 2e-3
        assert (dxb.sum(-1).abs() <= (4 * rtol) * gscale + 1e-6).all()
    rows = sample_rows(ab * s)
    sel = rows.to(device)
    xb, ob = x.view(ab * s, s)[sel].cpu(), out.view(ab * s, s)[sel].cpu()
    gb, dxb = g.view(ab * s, s)[sel].cpu(), dx.view(ab * s, s)[sel].cpu()
    qi = (rows % s).numpy()
    hidden = np.arange(s)[None, :] > qi[:, None]
    keep_rows = np.stack(
        [philox.keep_mask(s, p, seed, offset, first_element=int(r) * s) for r in rows]
    ).astype(bool)
    check(ob, cf.softmax_dropout_fwd(f64(xb), hidden, scale, keep_rows, p), name + " dropout fwd rows", atol=1e-9)
    check(dxb, cf.softmax_dropout_bwd(f64(gb), f64(xb), hidden, scale, keep_rows, p), name + " dropout bwd rows", atol=2e-7)


# --------------------------------------------------------------------------- cfg3
def test_padding_softmax_full_size(device):
    b, h, s = 16, 16, 1024
    scale = 0.125
    x = gpu_randn((b, h, s, s), F16, 3, device, std=2.0)
    g = gpu_randn((b, h, s, s), F16, 4, device)
    valid = torch.randint(256, 1025, (b,), generator=torch.Generator().manual_seed(3))
    pad = torch.arange(s)[None, :] >= valid[:, None]
    mask = pad.view(b, 1, 1, s).to(device)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x, mask, scale)
    dx = k.fused_scaled_masked_softmax_backward(g, y, scale, mask=mask)
    dx_dense = k.fused_scaled_masked_softmax_backward(g, y, scale)
    assert torch.equal(dx, dx_dense)
    for bi in range(b):
        yb = y[bi].float()
        assert (yb.sum(-1) - 1).abs().max().item() <= 2e-3
        assert yb[..., int(valid[bi]):].count_nonzero().item() == 0
        assert dx[bi][..., int(valid[bi]):].count_nonzero().item() == 0
    rows = sample_rows(b * h * s)
    sel = rows.to(device)
    xb, yb = x.view(-1, s)[sel].cpu(), y.view(-1, s)[sel].cpu()
    gb, dxb = g.view(-1, s)[sel].cpu(), dx.view(-1, s)[sel].cpu()
    bi = (rows // (h * s)).numpy()
    hidden = pad.numpy()[bi]
    check(yb, cf.softmax_masked_fwd(f64(xb), hidden, scale), "cfg3 fwd rows", atol=1e-9)
    check(dxb, cf.softmax_bwd(f64(gb), f64(yb), scale), "cfg3 bwd rows", atol=1e-7)


# --------------------------------------------------------------------------- cfg3 with the mask as an additive term
@pytest.mark.parametrize("kind", ["m10000", "inf", "position_bias"])
def test_additive_term_softmax_full_size(device, kind):
    """Configuration 3 with its mask in the form the reference's models pass
    it, an additive fp16 term [16, 1, 1, 1024] (-10000 as in
    oslo/transformers/models/bert/modeling_bert.py:298-306, and -inf), and with
    a dense position bias [1, 16, 1024, 1024]
    (oslo/transformers/models/t5/modeling_t5.py:508-514); with the dropout of
    the probabilities fused in as well."""
    b, h, s = 16, 16, 1024
    scale = 0.125
    x = gpu_randn((b, h, s, s), F16, 3, device, std=2.0)
    g = gpu_randn((b, h, s, s), F16, 4, device)
    valid = torch.randint(256, 1025, (b,), generator=torch.Generator().manual_seed(3))
    pad = torch.arange(s)[None, :] >= valid[:, None]
    if kind == "position_bias":
        term = gpu_randn((1, h, s, s), F16, 5, device, std=2.0)
    else:
        fill = -10000.0 if kind == "m10000" else float("-inf")
        term = torch.zeros(b, 1, 1, s, dtype=F16).masked_fill_(pad.view(b, 1, 1, s), fill).to(device)
    k = _C.get_softmax_kernel()
    y = k.softmax_bias_forward(x, term, scale)
    dx = k.softmax_bias_backward(g, y, scale, bias=term)
    assert torch.equal(dx, k.softmax_bias_backward(g, y, scale))
    for bi in range(b):
        yb = y[bi].float()
        assert (yb.sum(-1) - 1).abs().max().item() <= 2e-3
        if kind != "position_bias":
            assert yb[..., int(valid[bi]):].count_nonzero().item() == 0
            assert dx[bi][..., int(valid[bi]):].count_nonzero().item() == 0
        gscale = g[bi].float().abs().amax(-1) * scale
        assert (dx[bi].float().sum(-1).abs() <= 8e-3 * gscale + 1e-6).all()
    rows = sample_rows(b * h * s)
    sel = rows.to(device)
    xb, yb = x.view(-1, s)[sel].cpu(), y.view(-1, s)[sel].cpu()
    gb, dxb = g.view(-1, s)[sel].cpu(), dx.view(-1, s)[sel].cpu()
    bi, hi, qi = rows // (h * s), (rows // s) % h, rows % s
    tb = term.cpu()[0, hi, qi] if kind == "position_bias" else term.cpu()[bi, 0, 0]
    check(yb, cf.softmax_bias_fwd(f64(xb), f64(tb), scale), kind + " fwd rows", atol=1e-9)
    check(dxb, cf.softmax_bwd(f64(gb), f64(yb), scale), kind + " bwd rows", atol=1e-7)
    if kind != "position_bias":
        # the boolean-mask kernel on the same padding gives the same probabilities
        # (the two keep their logits in different domains: equal to an ulp)
        ym = k.fused_scaled_masked_softmax_forward(x, pad.view(b, 1, 1, s).to(device), scale)
        assert (y.float() - ym.float()).abs().max().item() <= 2.0 ** -10
        assert torch.equal(y == 0, ym == 0)
        del ym
    del dx, y
    p, seed, offset = 0.1, 321, 12
    out, stats = k.softmax_bias_dropout_forward(x, term, scale, p, seed, offset)
    dxd = k.softmax_bias_dropout_backward(g, x, term, stats, scale, p, seed, offset)
    ob, dxb = out.view(-1, s)[sel].cpu(), dxd.view(-1, s)[sel].cpu()
    keep_rows = np.stack(
        [philox.keep_mask(s, p, seed, offset, first_element=int(r) * s) for r in rows]
    ).astype(bool)
    check(ob, cf.softmax_bias_dropout_fwd(f64(xb), f64(tb), scale, keep_rows, p), kind + " dropout fwd rows",
          atol=1e-9)
    check(dxb, cf.softmax_bias_dropout_bwd(f64(gb), f64(xb), f64(tb), scale, keep_rows, p),
          kind + " dropout bwd rows", atol=2e-7)
    keep = _C.get_fused_elementwise_kernel().philox_mask(x.numel(), p, seed, offset, device).view(b, h, s, s)
    for bi in range(0, b, 4):
        assert out[bi:bi + 4][~keep[bi:bi + 4].bool()].count_nonzero().item() == 0


# --------------------------------------------------------------------------- cfg5 shape, causal + key padding
def test_causal_padding_softmax_full_size(device):
    """The attention of a causal model on a padded batch
    (oslo/transformers/models/gpt2/modeling_gpt2.py:126-136, 573-581) at the
    cfg5 shape: diagonal and key-padding mask in one call, with and without the
    fused dropout."""
    b, h, s = 4, 64, 2048
    scale = 1.0 / math.sqrt(96.0)
    x = gpu_randn((b, h, s, s), BF16, 11, device)
    g = gpu_randn((b, h, s, s), BF16, 12, device)
    valid = torch.randint(1024, 2049, (b,), generator=torch.Generator().manual_seed(5))
    pad = torch.arange(s)[None, :] >= valid[:, None]
    mask = pad.view(b, 1, 1, s).to(device)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x, mask, scale, causal=True)
    dx = k.fused_scaled_masked_softmax_backward(g, y, scale, mask=mask, causal=True)
    assert torch.equal(dx, k.fused_scaled_masked_softmax_backward(g, y, scale, causal=True))
    ar = torch.arange(1, s + 1, device=device)
    for bi in range(b):
        v = int(valid[bi])
        for h0 in range(0, h, 16):
            yb = y[bi, h0:h0 + 16].float()
            assert (yb.sum(-1) - 1).abs().max().item() <= 2e-3
            assert torch.triu(yb, diagonal=1).count_nonzero().item() == 0
            assert yb[..., v:].count_nonzero().item() == 0
            assert ((yb > 0).sum(-1) <= torch.clamp(ar, max=v)).all()
            dxb = dx[bi, h0:h0 + 16].float()
            assert torch.triu(dxb, diagonal=1).count_nonzero().item() == 0
            assert dxb[..., v:].count_nonzero().item() == 0
            gscale = g[bi, h0:h0 + 16].float().abs().amax(-1) * scale
            assert (dxb.sum(-1).abs() <= 8e-3 * gscale + 1e-6).all()
    rows = sample_rows(b * h * s)
    sel = rows.to(device)
    xb, yb = x.view(-1, s)[sel].cpu(), y.view(-1, s)[sel].cpu()
    gb, dxb = g.view(-1, s)[sel].cpu(), dx.view(-1, s)[sel].cpu()
    bi = (rows // (h * s)).numpy()
    qi = (rows % s).numpy()
    hidden = pad.numpy()[bi] | (np.arange(s)[None, :] > qi[:, None])
    check(yb, cf.softmax_masked_fwd(f64(xb), hidden, scale), "causal+padding fwd rows", atol=1e-9)
    check(dxb, cf.softmax_bwd(f64(gb), f64(yb), scale), "causal+padding bwd rows", atol=1e-7)
    del dx
    # with the dropout of the probabilities fused in
    p, seed, offset = 0.1, 777, 8
    out, stats = k.softmax_dropout_forward(x, mask, scale, p, seed, offset, causal=True)
    keep = _C.get_fused_elementwise_kernel().philox_mask(x.numel(), p, seed, offset, device).view(b, h, s, s)
    for bi in range(b):
        for h0 in range(0, h, 16):
            ob, yb, kb = out[bi, h0:h0 + 16].float(), y[bi, h0:h0 + 16].float(), keep[bi, h0:h0 + 16].bool()
            assert ob[~kb].count_nonzero().item() == 0
            want = yb / (1.0 - p)
            assert ((ob - want)[kb].abs() <= 2.0 ** -7 * want[kb] + 1e-30).all()
    del keep, y
    dxd = k.softmax_dropout_backward(g, x, stats, mask, scale, p, seed, offset, causal=True)
    ob, dxb = out.view(-1, s)[sel].cpu(), dxd.view(-1, s)[sel].cpu()
    keep_rows = np.stack(
        [philox.keep_mask(s, p, seed, offset, first_element=int(r) * s) for r in rows]
    ).astype(bool)
    check(ob, cf.softmax_dropout_fwd(f64(xb), hidden, scale, keep_rows, p), "causal+padding dropout fwd rows", atol=1e-9)
    check(dxb, cf.softmax_dropout_bwd(f64(gb), f64(xb), hidden, scale, keep_rows, p), "causal+padding dropout bwd rows",
          atol=2e-7)


# --------------------------------------------------------------------------- cfg2 / cfg5 norms
@pytest.mark.parametrize("n1,n2", [(16384, 4096), (8192, 6144)])
@pytest.mark.parametrize("rms", [False, True])
def test_norm_full_size(device, n1, n2, rms):
    eps = 1e-5
    x = gpu_randn((n1, n2), BF16, 5, device)
    dy = gpu_randn((n1, n2), BF16, 6, device)
    gamma = gpu_randn((n2,), BF16, 7, device, std=0.02, mean=1.0)
    beta = gpu_randn((n2,), BF16, 8, device, std=0.02)
    k = _C.get_layernorm_kernel()
    if rms:
        y, invvar = k.rms_norm_forward_affine(x, (n2,), gamma, eps)
        dx, dg = k.rms_norm_backward_affine(dy, invvar, x, (n2,), gamma, eps)
        mean = None
    else:
        y, mean, invvar = k.layer_norm_forward_affine(x, (n2,), gamma, beta, eps)
        dx, dg, db = k.layer_norm_backward_affine(dy, mean, invvar, x, (n2,), gamma, beta, eps)
    # (a) sampled rows
    rows = sample_rows(n1)
    sel = rows.to(device)
    xs, dys = f64(x[sel]), f64(dy[sel])
    if rms:
        oy, oinv = cf.rms_norm_fwd(xs, f64(gamma), eps, out="bf16")
        odx, _ = cf.rms_norm_bwd(dys, xs, oinv, f64(gamma))
        check(y[sel], np.asarray(oy, dtype=np.float64), "rms fwd rows", max_ulp=2, min_exact=0.995)
    else:
        oy, omean, oinv = cf.layer_norm_fwd(xs, f64(gamma), f64(beta), eps)
        odx, _, _ = cf.layer_norm_bwd(dys, xs, omean, oinv, f64(gamma))
        check(y[sel], oy, "ln fwd rows")
        assert np.allclose(f64(mean[sel]), omean, rtol=1e-5, atol=2e-6)
    assert np.allclose(f64(invvar[sel]), oinv, rtol=1e-5)
    check(dx[sel], odx, "norm bwd rows", atol=4e-6)
    # (b) whole-tensor: parameter gradients against float64 sums over all rows
    xh = np.empty((n1, n2), dtype=np.float64)
    dyf = np.empty((n1, n2), dtype=np.float64)
    step = 2048
    for s in range(0, n1, step):
        xb = f64(x[s:s + step])
        iv = f64(invvar[s:s + step])[:, None]
        mu = 0.0 if rms else f64(mean[s:s + step])[:, None]
        xh[s:s + step] = (xb - mu) * iv
        dyf[s:s + step] = f64(dy[s:s + step])
    odg = (dyf * xh).sum(0)
    check(dg, odg, "dgamma all rows", atol=1e-5 * math.sqrt(n1), min_exact=0.97)
    if not rms:
        check(db, dyf.sum(0), "dbeta all rows", atol=1e-5 * math.sqrt(n1), min_exact=0.97)
    # every row of dx: sum(dx * xhat) = 0 and (LayerNorm) sum(dx) = 0 up to rounding
    dxf = dx.float()
    bound = 4e-3 * dxf.abs().sum(-1) + 1e-3
    if not rms:
        assert (dxf.sum(-1).abs() <= bound).all()
    del dxf


# --------------------------------------------------------------------------- cfg4 / cfg5 bias-GeLU
@pytest.mark.parametrize("n1,n2", [(16384, 16384), (8192, 24576)])
def test_bias_gelu_full_size(device, n1, n2):
    x = gpu_randn((n1, n2), BF16, 9, device)
    g = gpu_randn((n1, n2), BF16, 10, device)
    bias = gpu_randn((n2,), BF16, 11, device, std=0.02)
    k = _C.get_fused_elementwise_kernel()
    y = k.bias_gelu_forward(x, bias)
    dx, db = k.bias_gelu_backward(g, x, bias)
    rows = sample_rows(n1, k=16)
    sel = rows.to(device)
    check(y[sel], cf.bias_gelu_fwd(f64(x[sel]), f64(bias)), "gelu fwd rows", atol=1e-6)
    check(dx[sel], cf.bias_gelu_bwd(f64(g[sel]), f64(x[sel]), f64(bias))[0], "gelu bwd rows", atol=1e-6)
    # whole tensor: gelu(u) in [-0.171, u+], and dbias = column sums of dx as stored
    assert torch.isfinite(y).all() and torch.isfinite(dx).all()
    assert (y.float().amin() >= -0.18)
    want = torch.zeros(n2, dtype=torch.float64, device=device)
    for s in range(0, n1, 2048):
        want += dx[s:s + 2048].double().sum(0)
    check(db, want.cpu().numpy(), "gelu dbias all rows", atol=1e-5 * math.sqrt(n1), min_exact=0.97)


# --------------------------------------------------------------------------- cfg4 / cfg5 bias-dropout-add
@pytest.mark.parametrize("n1,n2", [(16384, 4096), (8192, 6144)])
def test_bias_dropout_add_full_size(device, n1, n2):
    seed, offset, p = 1234, 0, 0.1
    x = gpu_randn((n1, n2), BF16, 12, device)
    res = gpu_randn((n1, n2), BF16, 13, device)
    g = gpu_randn((n1, n2), BF16, 14, device)
    bias = gpu_randn((n2,), BF16, 15, device, std=0.02)
    k = _C.get_fused_elementwise_kernel()
    # p = 0: exact
    out0 = k.bias_dropout_add_forward(x, bias, res, 0.0, seed, offset)
    assert torch.equal(out0, (x.float() + bias.float() + res.float()).to(BF16))
    dx0, db0 = k.bias_dropout_add_backward(g, 0.0, seed, offset)
    assert torch.equal(dx0, g)
    # p = 0.1: mask bit-exact on windows of the stream, values on sampled rows
    out, mask = k.bias_dropout_add_forward(x, bias, res, p, seed, offset, return_mask=True)
    flat = mask.view(-1)
    n = flat.numel()
    for start in (0, 4093 * n2 + 17, n - 100003):
        want = philox.keep_mask(100003, p, seed, offset, first_element=start)
        assert np.array_equal(flat[start:start + 100003].cpu().numpy(), want)
    keep_rate = flat.float().mean().item()
    assert abs(keep_rate - (1 - 6554 / 65536)) < 5 * math.sqrt(0.09 / n)
    rows = sample_rows(n1, k=16)
    sel = rows.to(device)
    keep = mask[sel].cpu().numpy()
    check(out[sel], cf.bias_dropout_add_fwd(f64(x[sel]), f64(bias), f64(res[sel]), keep, p), "bda fwd rows", atol=1e-6)
    dx, db = k.bias_dropout_add_backward(g, p, seed, offset)
    check(dx[sel], cf.bias_dropout_add_bwd(f64(g[sel]), keep, p)[0], "bda bwd rows", atol=1e-6)
    # whole tensor: dx is zero exactly where the mask says so; dbias = column sums
    assert torch.equal(dx == 0, (mask == 0) | (g == 0))
    want = dx.double().sum(0).cpu().numpy()
    check(db, want, "bda dbias all rows", atol=1e-5 * math.sqrt(n1), min_exact=0.97)
