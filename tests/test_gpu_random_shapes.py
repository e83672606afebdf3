"""Seeded random sweep over shapes, dtypes and option combinations of every op,
against the float64 oracle: ragged and odd row lengths, lengths around the
register-path limits, single rows, rows far apart in size, optional operands
on and off.  Complements the hand-picked cases of the other GPU test files."""
import os

import numpy as np
import pytest
import torch

from helpers import NP_NAME, check, f64, randn
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

# OSLO_FUZZ_SEED / OSLO_FUZZ_COUNT draw another (or a longer) sweep, e.g. for a soak run on new hardware:
# OSLO_FUZZ_SEED=7 OSLO_FUZZ_COUNT=500 pytest tests/test_gpu_random_shapes.py -m gpu
FUZZ_SEED = int(os.environ.get("OSLO_FUZZ_SEED", "0"))
FUZZ_COUNT = int(os.environ.get("OSLO_FUZZ_COUNT", "0"))

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
TRICKY = [1, 2, 3, 4, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513,
          520, 768, 1000, 1023, 1024, 1025, 1280, 1600, 2047, 2048, 2056, 4095, 4096, 4104, 5120, 8184, 8192,
          8200, 12288, 16376, 16384, 16392, 20000, 32768, 32776, 40000]


def draw_cases(seed, count):
    r = np.random.default_rng(seed + FUZZ_SEED)
    count = FUZZ_COUNT or count
    cases = []
    for i in range(count):
        n2 = int(r.choice(TRICKY)) if r.random() < 0.7 else int(r.integers(1, 9000))
        n1 = int(r.choice([1, 2, 3, 5, 8, 17, 33])) if n2 > 4096 else int(r.integers(1, 70))
        cases.append((i, n1, n2, DTYPES[int(r.integers(0, 3))], [bool(b) for b in r.integers(0, 2, size=4)]))
    return cases


@pytest.mark.parametrize("i,n1,n2,dtype,flags", draw_cases(101, 60))
def test_norms(device, i, n1, n2, dtype, flags):
    rms, affine = flags[0], flags[1]
    x = randn((n1, n2), dtype, 7 * i, std=1.5, mean=0.3)
    dy = randn((n1, n2), dtype, 7 * i + 1)
    gamma = randn((n2,), dtype, 7 * i + 2, std=0.1, mean=1.0) if affine else None
    beta = randn((n2,), dtype, 7 * i + 3, std=0.1) if affine and not rms else None
    k = _C.get_layernorm_kernel()
    name = NP_NAME[dtype]
    D = lambda t: None if t is None else t.to(device)
    col = 1e-5 * np.sqrt(n1) + 1e-6
    if rms:
        if affine:
            y, invvar = k.rms_norm_forward_affine(D(x), (n2,), D(gamma), 1e-5)
        else:
            y, invvar = k.rms_norm_forward(D(x), (n2,), 1e-5)
        oy, oinv = cf.rms_norm_fwd(f64(x), None if gamma is None else f64(gamma), 1e-5, name)
        check(y, oy, "rms fwd", atol=2e-6, max_ulp=2, min_exact=0.99)
        assert np.allclose(f64(invvar), oinv, rtol=3e-6)
        odx, odg = cf.rms_norm_bwd(f64(dy), f64(x), f64(invvar), None if gamma is None else f64(gamma))
        if affine:
            dx, dg = k.rms_norm_backward_affine(D(dy), invvar, D(x), (n2,), D(gamma), 1e-5)
            check(dg, odg, "rms dgamma", atol=col, min_exact=0.97, max_ulp=2)
        else:
            dx = k.rms_norm_backward(D(dy), invvar, D(x), (n2,), 1e-5)
        amp = float(np.abs(f64(invvar)).max()) * float(np.abs(f64(dy)).max()) * (
            1.0 if gamma is None else float(np.abs(f64(gamma)).max()))
        check(dx, odx, "rms dx", atol=4e-6 + 2.5e-7 * amp)
    else:
        if affine:
            y, mean, invvar = k.layer_norm_forward_affine(D(x), (n2,), D(gamma), D(beta), 1e-5)
        else:
            y, mean, invvar = k.layer_norm_forward(D(x), (n2,), 1e-5)
        oy, omean, oinv = cf.layer_norm_fwd(f64(x), None if gamma is None else f64(gamma),
                                            None if beta is None else f64(beta), 1e-5)
        # a row of one element (or of equal elements) normalises to ~0: absolute floor
        check(y, oy, "ln fwd", atol=2e-5)
        assert np.allclose(f64(mean), omean, rtol=1e-5, atol=2e-6)
        if n2 > 1:
            assert np.allclose(f64(invvar), oinv, rtol=1e-4)
        odx, odg, odb = cf.layer_norm_bwd(f64(dy), f64(x), f64(mean), f64(invvar),
                                          None if gamma is None else f64(gamma))
        if affine:
            dx, dg, db = k.layer_norm_backward_affine(D(dy), mean, invvar, D(x), (n2,), D(gamma), D(beta), 1e-5)
            check(dg, odg, "ln dgamma", atol=col * 3, min_exact=0.97, max_ulp=2)
            check(db, odb, "ln dbeta", atol=col, min_exact=0.97, max_ulp=2)
        else:
            dx = k.layer_norm_backward(D(dy), mean, invvar, D(x), (n2,), 1e-5)
        amp = float(np.abs(f64(invvar)).max()) * float(np.abs(f64(dy)).max()) * (
            1.0 if gamma is None else float(np.abs(f64(gamma)).max()))
        check(dx, odx, "ln dx", atol=2e-5 + 2.5e-7 * amp)  # (rounding amplified by invvar, see the fused test)


@pytest.mark.parametrize("i,n1,n2,dtype,flags", draw_cases(202, 50))
def test_fused_residual_norm(device, i, n1, n2, dtype, flags):
    rms, has_bias, has_res, has_extra = flags
    p = [0.0, 0.1, 0.5][i % 3]
    seed, offset = 1000 + i, 4 * i
    x = randn((n1, n2), dtype, 11 * i)
    bias = randn((n2,), dtype, 11 * i + 1, std=0.1) if has_bias else None
    res = randn((n1, n2), dtype, 11 * i + 2) if has_res else None
    gamma = randn((n2,), dtype, 11 * i + 3, std=0.1, mean=1.0)
    beta = None if rms else randn((n2,), dtype, 11 * i + 4, std=0.1)
    dy = randn((n1, n2), dtype, 11 * i + 5)
    dh = randn((n1, n2), dtype, 11 * i + 6) if has_extra else None
    k = _C.get_layernorm_kernel()
    name = NP_NAME[dtype]
    D = lambda t: None if t is None else t.to(device)
    F = lambda t: None if t is None else f64(t)
    y, h, mean, invvar = k.bias_dropout_add_norm_forward(
        rms, D(x), D(bias), D(res), (n2,), D(gamma), D(beta), 1e-5, p, seed, offset)
    keep = philox.keep_mask(n1 * n2, p, seed, offset).reshape(n1, n2).astype(bool) if p > 0 else None
    # (three fp32 roundings before the store: ties fall the other way a little
    # more often than the default 0.2 %)
    check(h, cf.bias_dropout_add_fwd(f64(x), F(bias), F(res), keep, p), "fused h", atol=1e-6, min_exact=0.99)
    if rms:
        oy, _ = cf.rms_norm_fwd(f64(h), f64(gamma), 1e-5, name)
    else:
        oy, _, _ = cf.layer_norm_fwd(f64(h), f64(gamma), f64(beta), 1e-5, name)
    check(y, oy, "fused y", atol=2e-5, max_ulp=2, min_exact=0.99)
    g_res, g_in, g_gamma, g_beta, g_bias = k.bias_dropout_add_norm_backward(
        rms, D(dy), D(dh), h, mean, invvar, (n2,), D(gamma), p, seed, offset, need_bias_grad=has_bias)
    odres, odx, odg, odb, _ = cf.bias_dropout_add_norm_bwd(
        f64(dy), F(dh), f64(h), None if rms else f64(mean), f64(invvar), f64(gamma), keep, p, rms, name)
    # fp32 rounding of dy * gamma is amplified by invvar: a row of one element (or of equal elements) has
    # invvar = 1 / sqrt(eps) = 316 and a gradient that cancels to 0 exactly only in exact arithmetic
    amp = float(np.abs(f64(invvar)).max()) * float(np.abs(f64(dy)).max()) * float(np.abs(f64(gamma)).max())
    atol_dx = 2e-5 + 2.5e-7 * amp
    check(g_res, odres, "fused dres", atol=atol_dx)
    check(g_in, odx, "fused dx", atol=atol_dx)
    col = 1e-5 * np.sqrt(n1) + 1e-6
    check(g_gamma, odg, "fused dgamma", atol=3 * col, min_exact=0.97, max_ulp=2)
    if has_bias:
        check(g_bias, f64(g_in).sum(0), "fused dbias", atol=3 * col, min_exact=0.97, max_ulp=2)


def draw_softmax(seed, count):
    r = np.random.default_rng(seed + FUZZ_SEED)
    count = FUZZ_COUNT or count
    out = []
    for i in range(count):
        sk = int(r.choice([1, 5, 8, 16, 31, 64, 100, 128, 256, 257, 512, 1000, 1024, 2048, 2050, 4096, 8192, 9000,
                           16384, 20000]))
        sq = int(r.integers(1, 40)) if r.random() < 0.6 else min(sk, 48)
        b, np_ = int(r.integers(1, 4)), int(r.integers(1, 4))
        out.append((i, b, np_, sq, sk, DTYPES[int(r.integers(0, 3))], int(r.integers(0, 7))))
    return out


@pytest.mark.parametrize("i,b,np_,sq,sk,dtype,kind", draw_softmax(303, 60))
def test_softmax_with_and_without_dropout(device, i, b, np_, sq, sk, dtype, kind):
    """kind 0: causal; 1: key padding; 2: per-query mask; 3: shared mask; 4: rows fully masked;
    5: causal + key padding in one call; 6: causal + per-query mask in one call."""
    r = np.random.default_rng(1000 + i)
    scale = float(r.choice([0.125, 0.5, 1.0]))
    p = float(r.choice([0.0, 0.1, 0.3]))
    seed, offset = 50 + i, 4 * i
    x = randn((b, np_, sq, sk), dtype, 13 * i, std=2.0)
    g = randn((b, np_, sq, sk), dtype, 13 * i + 1)
    k = _C.get_softmax_kernel()
    causal = kind >= 5
    if kind == 0:
        hidden = cf.causal_hidden(sq, sk)
        mask = None
        xin, gin = x.view(b * np_, sq, sk), g.view(b * np_, sq, sk)
    else:
        if kind in (1, 5):
            valid = r.integers(1, sk + 1, size=b)
            m = np.arange(sk)[None, :] >= valid[:, None]
            mask = torch.from_numpy(m).view(b, 1, 1, sk)
        elif kind in (2, 6):
            m = r.random((b, 1, sq, sk)) < 0.4
            m[..., 0] = False
            mask = torch.from_numpy(m)
        elif kind == 3:
            m = r.random((1, 1, sq, sk)) < 0.4
            m[..., 0] = False
            mask = torch.from_numpy(m)
        else:
            m = r.random((b, 1, sq, sk)) < 0.3
            m[:, :, ::2, :] = True
            mask = torch.from_numpy(m)
        hidden = mask.numpy()
        if causal:
            hidden = hidden | cf.causal_hidden(sq, sk)[None, None]
        xin, gin = x, g
    xd, gd = xin.to(device), gin.to(device)
    md = None if mask is None else mask.to(device)
    xv, gv = f64(xin), f64(gin)
    if p == 0.0:
        if mask is None:
            y = k.fused_scaled_upper_triang_masked_softmax_forward(xd, scale)
            dx = k.fused_scaled_upper_triang_masked_softmax_backward(gd, y, scale)
        else:
            y = k.fused_scaled_masked_softmax_forward(xd, md, scale, causal=causal)
            dx = k.fused_scaled_masked_softmax_backward(gd, y, scale, mask=md, causal=causal)
        check(y, cf.softmax_masked_fwd(xv, hidden, scale), "softmax fwd", atol=1e-9)
        check(dx, cf.softmax_bwd(gv, f64(y), scale), "softmax bwd", atol=2e-7)
    else:
        out, stats = k.softmax_dropout_forward(xd, md, scale, p, seed, offset, causal=causal)
        keep = philox.keep_mask(x.numel(), p, seed, offset).reshape(xv.shape).astype(bool)
        check(out, cf.softmax_dropout_fwd(xv, hidden, scale, keep, p), "softmax dropout fwd", atol=1e-9)
        dx = k.softmax_dropout_backward(gd, xd, stats, md, scale, p, seed, offset, causal=causal)
        # (the dropped elements of a row share one gradient value, -scale * y * sum; when that value is a
        #  rounding tie of the storage type, which 16-bit inputs and a uniform row of 1 / sk make likely,
        #  every one of them lands on the other side: a handful of 1-ulp differences in a tensor this small)
        check(dx, cf.softmax_dropout_bwd(gv, xv, hidden, scale, keep, p), "softmax dropout bwd", atol=3e-7,
              min_exact=0.98)


def draw_term_softmax(seed, count):
    r = np.random.default_rng(seed + FUZZ_SEED)
    count = FUZZ_COUNT or count
    out = []
    for i in range(count):
        sk = int(r.choice([1, 5, 8, 16, 24, 31, 64, 96, 100, 128, 192, 256, 257, 384, 512, 768, 1000, 1024, 1536,
                           2048, 2050, 4096, 8192, 9000, 16384]))
        sq = int(r.integers(1, 40)) if r.random() < 0.6 else min(sk, 48)
        b, np_ = int(r.integers(1, 5)), int(r.integers(1, 4))
        out.append((i, b, np_, sq, sk, DTYPES[int(r.integers(0, 3))], int(r.integers(0, 6))))
    return out


@pytest.mark.parametrize("i,b,np_,sq,sk,dtype,kind", draw_term_softmax(505, 60))
def test_softmax_with_an_additive_term(device, i, b, np_, sq, sk, dtype, kind):
    """kind 0: -10000 key mask [b,1,1,sk]; 1: lowest-value key mask; 2: -inf staircase per query
    [b,1,sq,sk] (key 0 stays visible); 3: dense term shared by the batch [1,np,sq,sk]; 4: dense
    term per sample and head; 5: per-head vector [np,1,sk].  Each with or without the diagonal,
    the term in the scores' type or in float32, hidden chunks skipped or not, with or without
    the fused dropout."""
    r = np.random.default_rng(2000 + i)
    scale = float(r.choice([0.125, 0.5, 1.0]))
    p = float(r.choice([0.0, 0.0, 0.1, 0.3]))
    causal = bool(r.integers(0, 2))   # (with sq > sk the first sq - sk queries see no key at all)
    skip = bool(r.integers(0, 2))
    term_f32 = bool(r.integers(0, 2))
    seed, offset = 70 + i, 4 * i
    x = randn((b, np_, sq, sk), dtype, 19 * i, std=2.0)
    g = randn((b, np_, sq, sk), dtype, 19 * i + 1)
    tdtype = torch.float32 if term_f32 else dtype
    if kind in (0, 1):
        valid = r.integers(1, sk + 1, size=b)
        pad = torch.from_numpy(np.arange(sk)[None, :] >= valid[:, None]).view(b, 1, 1, sk)
        fill = -10000.0 if kind == 0 else float(torch.finfo(tdtype).min)
        term = torch.zeros(b, 1, 1, sk).masked_fill(pad, fill).to(tdtype)
    elif kind == 2:
        cut = torch.from_numpy(r.integers(1, sk + 1, size=(b, 1, sq, 1)))
        term = torch.zeros(b, 1, sq, sk).masked_fill(
            torch.arange(sk).view(1, 1, 1, sk) >= cut, float("-inf")).to(tdtype)
    elif kind == 3:
        term = randn((1, np_, sq, sk), tdtype, 19 * i + 2, std=2.0)
    elif kind == 4:
        term = randn((b, np_, sq, sk), tdtype, 19 * i + 2, std=2.0)
    else:
        term = randn((np_, 1, sk), tdtype, 19 * i + 2, std=2.0)
    k = _C.get_softmax_kernel()
    xd, gd, td = x.to(device), g.to(device), term.to(device)
    xv, gv, tv = f64(x), f64(g), f64(term)
    # a query that the diagonal leaves without any key is NaN in the oracle (as in torch) and zeros here
    seen = np.ones((b, np_, sq), dtype=bool)
    if causal and sq > sk:
        seen[..., : sq - sk] = False
    st = torch.from_numpy(seen)

    def compare(actual, truth, what, **kw):
        a = actual.cpu()
        assert (a[~st] == 0).all(), what + ": a query without any key must come out as zeros"
        if seen.any():
            check(a[st], truth[seen], what, **kw)

    if p == 0.0:
        y = k.softmax_bias_forward(xd, td, scale, causal=causal, skip_hidden=skip)
        dx = k.softmax_bias_backward(gd, y, scale, bias=td, causal=causal, skip_hidden=skip)
        compare(y, cf.softmax_bias_fwd(xv, tv, scale, causal=causal), "term softmax fwd", atol=1e-9)
        compare(dx, cf.softmax_bwd(gv, f64(y), scale), "term softmax bwd", atol=2e-7)
    else:
        out, stats = k.softmax_bias_dropout_forward(xd, td, scale, p, seed, offset, causal=causal,
                                                    skip_hidden=skip)
        assert torch.isfinite(stats).all()
        keep = philox.keep_mask(x.numel(), p, seed, offset).reshape(xv.shape).astype(bool)
        compare(out, cf.softmax_bias_dropout_fwd(xv, tv, scale, keep, p, causal=causal),
                "term softmax dropout fwd", atol=1e-9)
        dx = k.softmax_bias_dropout_backward(gd, xd, td, stats, scale, p, seed, offset, causal=causal,
                                             skip_hidden=skip)
        # dx = scale * y * (dp - sum(dp * y)) cancels: the absolute floor is two float32 roundings of the
        # largest product scale * y * dp that can enter it (y <= 1)
        floor = max(3e-7, 2 * 2.0 ** -23 * scale * float(np.abs(gv).max()) / (1.0 - p))
        compare(dx, cf.softmax_bias_dropout_bwd(gv, xv, tv, scale, keep, p, causal=causal),
                "term softmax dropout bwd", atol=floor, min_exact=0.98)


@pytest.mark.parametrize("i,n1,n2,dtype,flags", draw_cases(404, 50))
def test_elementwise(device, i, n1, n2, dtype, flags):
    has_bias, has_res = flags[0], flags[1]
    p = [0.0, 0.1, 0.6][i % 3]
    seed, offset = 9 + i, 4 * i
    x = randn((n1, n2), dtype, 17 * i, std=1.5)
    g = randn((n1, n2), dtype, 17 * i + 1)
    bias = randn((n2,), dtype, 17 * i + 2, std=0.3) if has_bias else None
    res = randn((n1, n2), dtype, 17 * i + 3) if has_res else None
    k = _C.get_fused_elementwise_kernel()
    name = NP_NAME[dtype]
    D = lambda t: None if t is None else t.to(device)
    F = lambda t: None if t is None else f64(t)
    col = 1e-5 * np.sqrt(n1) + 1e-6
    y = k.bias_gelu_forward(D(x), D(bias))
    check(y, cf.bias_gelu_fwd(f64(x), F(bias)), "gelu fwd", atol=1e-6)
    dx, db = k.bias_gelu_backward(D(g), D(x), D(bias), need_bias_grad=has_bias)
    odx, _ = cf.bias_gelu_bwd(f64(g), f64(x), F(bias), out=name)
    check(dx, cf.bias_gelu_bwd(f64(g), f64(x), F(bias))[0], "gelu bwd", atol=1e-6)
    if has_bias:
        check(db, f64(dx).sum(0), "gelu dbias", atol=3 * col, min_exact=0.97, max_ulp=2)
    out = k.bias_dropout_add_forward(D(x), D(bias), D(res), p, seed, offset)
    keep = philox.keep_mask(n1 * n2, p, seed, offset).reshape(n1, n2).astype(bool) if p > 0 else None
    check(out, cf.bias_dropout_add_fwd(f64(x), F(bias), F(res), keep, p), "bda fwd", atol=1e-6, min_exact=0.99)
    ddx, ddb = k.bias_dropout_add_backward(D(g), p, seed, offset, need_bias_grad=has_bias)
    check(ddx, cf.bias_dropout_add_bwd(f64(g), keep, p)[0], "bda bwd", atol=1e-6)
    if has_bias:
        check(ddb, f64(ddx).sum(0), "bda dbias", atol=3 * col, min_exact=0.97, max_ulp=2)
