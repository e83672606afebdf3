"""Pins the numpy oracle (oracle/closed_form.py) without a GPU: against torch's
library routines and autograd in float64, against finite differences, and
against the invariants the mathematics fixes.  Each check is chosen so that a
dropped term, a wrong sign or a transposed operand fails it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import closed_form as cf
from oracle import torch_path as tp


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- rounding
def test_round_bf16_matches_torch():
    a = rng(0).standard_normal(100000).astype(np.float32) * 37.0
    a[:8] = [0.0, -0.0, 1.0, 1.00390625, 1.001953125, 1.005859375, 3.0e38, 1e-40]
    got = cf.round_bf16(a)
    want = torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_round_f16_matches_torch():
    a = rng(1).standard_normal(100000).astype(np.float32) * 11.0
    got = cf.round_f16(a)
    want = torch.from_numpy(a).to(torch.float16).to(torch.float32).numpy()
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- softmax
@pytest.mark.parametrize("sq,sk", [(1, 1), (5, 5), (3, 7), (7, 3), (16, 16)])
def test_causal_softmax_vs_torch_where_chain(sq, sk):
    x = rng(2).standard_normal((3, sq, sk))
    y = cf.softmax_causal_fwd(x, 0.37)
    ref = tp.causal_softmax(torch.from_numpy(x), 0.37).numpy() if sq <= sk else None
    if ref is not None:
        # the -1e4 fill of the reference underflows to exactly 0 in the softmax
        assert np.allclose(y, ref, rtol=1e-12, atol=0)
        assert np.array_equal(y == 0, ref == 0)
    hidden = cf.causal_hidden(sq, sk)
    rows_visible = (~hidden).sum(-1)
    # hidden keys are exactly 0 in every row that sees at least one key
    assert np.all(y[:, hidden & (rows_visible > 0)[:, None]] == 0)
    assert np.allclose(y.sum(-1)[:, rows_visible > 0], 1.0, atol=1e-14)
    # query i sees exactly i + 1 + (sk - sq) keys
    want_nz = np.clip(np.arange(sq) + 1 + (sk - sq), 0, sk)
    got_nz = (y[0] > 0).sum(-1)
    assert np.array_equal(got_nz[want_nz > 0], want_nz[want_nz > 0])
    # no visible key: uniform
    assert np.allclose(y[:, want_nz == 0], 1.0 / sk)
    if sq == sk:
        assert np.all(y[:, 0, 0] == 1.0)


def test_masked_softmax_vs_torch_additive_mask():
    b, h, sq, sk = 3, 2, 4, 12
    x = rng(3).standard_normal((b, h, sq, sk)) * 2
    valid = np.array([12, 5, 1])
    pad = np.arange(sk)[None, :] >= valid[:, None]
    y = cf.softmax_masked_fwd(x, pad[:, None, None, :], 0.125)
    ref = tp.padding_softmax(torch.from_numpy(x), torch.from_numpy(pad), 0.125).numpy()
    assert np.allclose(y, ref, rtol=1e-12, atol=0)
    assert np.all(y[np.broadcast_to(pad[:, None, None, :], y.shape)] == 0)
    # masked_fill(-inf) variant (DistilBERT) is the same function
    t = torch.from_numpy(x * 0.125).masked_fill(torch.from_numpy(pad)[:, None, None, :], -np.inf)
    assert np.allclose(y, torch.softmax(t, -1).numpy(), rtol=1e-12, atol=0)


def test_masked_softmax_fully_masked_row_is_uniform():
    x = rng(4).standard_normal((1, 1, 2, 8))
    hidden = np.zeros((1, 1, 2, 8), dtype=bool)
    hidden[0, 0, 1, :] = True
    y = cf.softmax_masked_fwd(x, hidden, 1.0)
    assert np.allclose(y[0, 0, 1], 1 / 8)
    t = torch.from_numpy(x).masked_fill(torch.from_numpy(hidden), -10000.0)
    assert np.allclose(y, torch.softmax(t, -1).numpy(), rtol=1e-12)


def test_softmax_shift_invariance_and_scale():
    x = rng(5).standard_normal((2, 6, 6))
    a = cf.softmax_causal_fwd(x, 0.5)
    b = cf.softmax_causal_fwd(x + 3.25, 0.5)
    assert np.allclose(a, b, rtol=1e-12, atol=1e-16)
    c = cf.softmax_causal_fwd(2 * x, 0.25)
    assert np.allclose(a, c, rtol=1e-12, atol=1e-16)


def test_softmax_bwd_vs_autograd_and_row_sum():
    x = torch.from_numpy(rng(6).standard_normal((2, 5, 9))).requires_grad_()
    g = torch.from_numpy(rng(7).standard_normal((2, 5, 9)))
    scale = 0.3
    y = tp.causal_softmax(x, scale)
    y.backward(g)
    dx = cf.softmax_bwd(g.numpy(), y.detach().numpy(), scale)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-10, atol=1e-14)
    assert np.allclose(dx.sum(-1), 0, atol=1e-14)
    # dropping the scale or the row sum must be visible
    assert not np.allclose(cf.softmax_bwd(g.numpy(), y.detach().numpy(), 1.0), x.grad.numpy())


# ------------------------------------------ softmax with an additive term
@pytest.mark.parametrize("bias_shape", [(3, 1, 1, 12), (1, 4, 5, 12), (3, 4, 5, 12), (1, 1, 5, 12)])
def test_bias_softmax_vs_torch_additive_chain_and_autograd(bias_shape):
    """torch.softmax(scale * x + M) in float64 and its autograd: forward, the
    gradient of x (scale * y * (g - sum g y)) and, through it, the gradient
    of M (the same without the scale, summed over the broadcast dimensions)."""
    r = rng(40)
    x = torch.from_numpy(r.standard_normal((3, 4, 5, 12)) * 2).requires_grad_()
    m = torch.from_numpy(r.standard_normal(bias_shape) * 3).requires_grad_()
    g = torch.from_numpy(r.standard_normal((3, 4, 5, 12)))
    scale = 0.37
    y = torch.softmax(scale * x + m, dim=-1)
    y.backward(g)
    oy = cf.softmax_bias_fwd(x.detach().numpy(), m.detach().numpy(), scale, sum_f32=False)
    assert np.allclose(oy, y.detach().numpy(), rtol=1e-12, atol=0)
    dx = cf.softmax_bwd(g.numpy(), oy, scale)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-10, atol=1e-14)
    dm = (dx / scale).reshape(3, 4, 5, 12)
    for d, size in enumerate(bias_shape[:3]):
        if size == 1:
            dm = dm.sum(axis=d, keepdims=True)
    assert np.allclose(dm, m.grad.numpy(), rtol=1e-10, atol=1e-13)
    # rounding the sum to float32 moves a probability by a few float32 ulps of the logit
    assert np.allclose(cf.softmax_bias_fwd(x.detach().numpy(), m.detach().numpy(), scale), oy,
                       rtol=2e-6, atol=0)
    # a transposed or dropped term must be visible
    assert not np.allclose(cf.softmax_bias_fwd(x.detach().numpy(), 0.0, scale), oy, rtol=1e-3)


def test_bias_softmax_padding_conventions_of_the_reference():
    """The -10000 mask of modeling_bert.py / modeling_gpt2.py, the finfo.min
    mask of modeling_bart.py and a -inf mask against the boolean-mask oracle
    (pinned above) wherever a row sees a key; and the three conventions on a
    row that sees none, against torch in float32."""
    b, h, sq, sk = 3, 2, 4, 16
    r = rng(41)
    x = r.standard_normal((b, h, sq, sk)).astype(np.float32) * 2
    valid = np.array([16, 5, 1])
    pad = np.arange(sk)[None, :] >= valid[:, None]
    want = cf.softmax_masked_fwd(x, pad[:, None, None, :], 0.125)
    for fill in (-10000.0, float(np.finfo(np.float32).min), -np.inf,
                 float(torch.finfo(torch.bfloat16).min), -65504.0):
        m = np.where(pad, fill, 0.0)[:, None, None, :]
        y = cf.softmax_bias_fwd(x, m, 0.125)
        assert np.allclose(y, want, rtol=1e-6, atol=0), fill
        assert np.all(y[np.broadcast_to(pad[:, None, None, :], y.shape)] == 0), fill
    # rows without a visible key
    xt = torch.from_numpy(x[:1, :1])
    full = lambda v: torch.full((1, 1, 1, sk), v, dtype=torch.float32)
    # -10000 everywhere: the softmax of the logits themselves (the float32 sum keeps
    # the logit to 2^-10, hence the tolerance: torch rounds the product first)
    y = cf.softmax_bias_fwd(x[:1, :1], full(-10000.0).numpy(), 0.125)
    assert np.allclose(y, torch.softmax(xt * 0.125 + full(-10000.0), -1).numpy(), rtol=2e-3)
    assert np.allclose(y, cf.softmax_masked_fwd(x[:1, :1], False, 0.125), rtol=2e-3)
    assert not np.allclose(y, 1.0 / sk, rtol=0.05)
    # the lowest float everywhere: it absorbs the logit, the row is uniform
    lo = float(np.finfo(np.float32).min)
    y = cf.softmax_bias_fwd(x[:1, :1], full(lo).numpy(), 0.125)
    assert np.array_equal(y, torch.softmax(xt * 0.125 + full(lo), -1).double().numpy())
    assert np.all(y == 1.0 / sk)
    # the lowest float16 does not absorb a float32 logit: the row is the softmax of
    # the logits, coarsely (the sum keeps them to 2^-8)
    y = cf.softmax_bias_fwd(x[:1, :1], full(-65504.0).numpy(), 0.125)
    assert np.allclose(y, cf.softmax_masked_fwd(x[:1, :1], False, 0.125), rtol=5e-3)
    assert not np.allclose(y, 1.0 / sk, rtol=0.05)
    # -inf everywhere: NaN, as torch returns
    y = cf.softmax_bias_fwd(x[:1, :1], full(-np.inf).numpy(), 0.125)
    assert np.isnan(y).all()
    assert torch.isnan(torch.softmax(xt * 0.125 + full(-np.inf), -1)).all()
    # -inf and the lowest float mixed: uniform over the finite ones
    m = full(lo).numpy().copy()
    m[..., ::2] = -np.inf
    y = cf.softmax_bias_fwd(x[:1, :1], m, 0.125)
    assert np.array_equal(y, torch.softmax(xt * 0.125 + torch.from_numpy(m), -1).double().numpy())
    assert np.all(y[..., 1::2] == 2.0 / sk) and np.all(y[..., ::2] == 0)


def test_bias_softmax_causal_flag_is_a_minus_inf_triangle():
    r = rng(42)
    for sq, sk in ((6, 6), (3, 9), (1, 5)):
        x = r.standard_normal((2, 3, sq, sk))
        m = r.standard_normal((1, 3, sq, sk))
        tri = np.where(cf.causal_hidden(sq, sk), -np.inf, 0.0)
        y = cf.softmax_bias_fwd(x, m, 0.5, causal=True, sum_f32=False)
        ref = torch.softmax(torch.from_numpy(0.5 * x + m + tri), -1).numpy()
        assert np.allclose(y, ref, rtol=1e-12, atol=0)
        assert np.all(y[..., cf.causal_hidden(sq, sk)] == 0)
        # without a term the causal softmax (pinned above)
        assert np.allclose(cf.softmax_bias_fwd(x.reshape(6, sq, sk)[None], 0.0, 0.5, causal=True,
                                               sum_f32=False)[0],
                           cf.softmax_causal_fwd(x.reshape(6, sq, sk), 0.5), rtol=1e-12, atol=0)


def test_bias_softmax_dropout_vs_autograd():
    r = rng(43)
    x = torch.from_numpy(r.standard_normal((2, 3, 4, 8))).requires_grad_()
    m = torch.from_numpy(r.standard_normal((1, 3, 4, 8)))
    g = torch.from_numpy(r.standard_normal((2, 3, 4, 8)))
    keep = r.random((2, 3, 4, 8)) >= 0.25
    p, scale = 0.25, 0.7
    ps = float(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))
    out = torch.softmax(scale * x + m, -1) * torch.from_numpy(keep) * ps
    out.backward(g)
    o = cf.softmax_bias_dropout_fwd(x.detach().numpy(), m.numpy(), scale, keep, p)
    # (the float32 sum of the oracle: a few float32 ulps of the logits)
    assert np.allclose(o, out.detach().numpy(), rtol=2e-6, atol=0)
    dx = cf.softmax_bias_dropout_bwd(g.numpy(), x.detach().numpy(), m.numpy(), scale, keep, p)
    assert np.allclose(dx, x.grad.numpy(), rtol=2e-5, atol=1e-7)
    # p = 0 without a keep mask is the plain pair
    assert np.array_equal(cf.softmax_bias_dropout_fwd(x.detach().numpy(), m.numpy(), scale, None, 0.0),
                          cf.softmax_bias_fwd(x.detach().numpy(), m.numpy(), scale))


# ---------------------------------------------------------------- norms
@pytest.mark.parametrize("n2", [1, 7, 64, 513])
def test_layer_norm_fwd_bwd_vs_torch_fp64(n2):
    r = rng(8 + n2)
    x = torch.from_numpy(r.standard_normal((6, n2)) * 1.7 + 0.4).requires_grad_()
    w = torch.from_numpy(1 + 0.1 * r.standard_normal(n2)).requires_grad_()
    b = torch.from_numpy(0.1 * r.standard_normal(n2)).requires_grad_()
    g = torch.from_numpy(r.standard_normal((6, n2)))
    eps = 1e-5
    y = F.layer_norm(x, (n2,), w, b, eps)
    y.backward(g)
    oy, mean, invvar = cf.layer_norm_fwd(x.detach().numpy(), w.detach().numpy(), b.detach().numpy(), eps)
    assert np.allclose(oy, y.detach().numpy(), rtol=1e-11, atol=1e-13)
    assert np.allclose(mean, x.detach().numpy().mean(-1))
    assert np.allclose(invvar, 1 / np.sqrt(x.detach().numpy().var(-1) + eps))
    dx, dg, db = cf.layer_norm_bwd(g.numpy(), x.detach().numpy(), mean, invvar, w.detach().numpy())
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-9, atol=1e-11)
    assert np.allclose(dg, w.grad.numpy(), rtol=1e-10, atol=1e-12)
    assert np.allclose(db, b.grad.numpy(), rtol=1e-10, atol=1e-12)
    assert np.allclose(db, g.numpy().sum(0))


def test_layer_norm_invariants():
    r = rng(20)
    x = r.standard_normal((5, 96)) * 3 + 1
    g = r.standard_normal((5, 96))
    eps = 1e-5
    y, mean, invvar = cf.layer_norm_fwd(x, None, None, eps)
    assert np.allclose(y.mean(-1), 0, atol=1e-14)
    var = x.var(-1)
    assert np.allclose(y.var(-1), var / (var + eps), rtol=1e-12)
    dx, dg, db = cf.layer_norm_bwd(g, x, mean, invvar, None)
    assert dg is None and db is None
    assert np.allclose(dx.sum(-1), 0, atol=1e-13)
    # sum(dx * xhat) vanishes up to the factor eps / (var + eps) ~ 1e-6
    assert np.allclose((dx * y).sum(-1), 0, atol=1e-4)
    dx0, _, _ = cf.layer_norm_bwd(g, x, mean, 1 / np.sqrt(x.var(-1)), None)
    y0 = (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True))
    assert np.allclose((dx0 * y0).sum(-1), 0, atol=1e-12)


@pytest.mark.parametrize("n2", [1, 8, 200])
def test_rms_norm_fwd_bwd_vs_autograd_fp64(n2):
    r = rng(30 + n2)
    x = torch.from_numpy(r.standard_normal((4, n2)) + 0.3).requires_grad_()
    w = torch.from_numpy(1 + 0.1 * r.standard_normal(n2)).requires_grad_()
    g = torch.from_numpy(r.standard_normal((4, n2)))
    eps = 1e-6
    # manual_rms_norm takes the variance in fp32 whatever the input type
    # (layer_norm.py:20), so the reference path itself pins only ~1e-7; the
    # same formula without that cast pins the rest of the digits
    y = w * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))
    y.backward(g)
    oy, invvar = cf.rms_norm_fwd(x.detach().numpy(), w.detach().numpy(), eps)
    assert np.allclose(oy, y.detach().numpy(), rtol=1e-12, atol=1e-14)
    assert np.allclose(oy, tp.rms_norm(x.detach(), w.detach(), eps).numpy(), rtol=1e-6)
    dx, dg = cf.rms_norm_bwd(g.numpy(), x.detach().numpy(), invvar, w.detach().numpy())
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-9, atol=1e-12)
    assert np.allclose(dg, w.grad.numpy(), rtol=1e-10, atol=1e-12)
    xhat = x.detach().numpy() * invvar[:, None]
    dx0, _ = cf.rms_norm_bwd(g.numpy(), x.detach().numpy(), invvar, None)
    if n2 > 1:
        # exact only for eps -> 0; eps = 1e-6 leaves a 1e-6-relative residue
        assert np.allclose((dx0 * xhat).sum(-1), 0, atol=1e-4)


def test_rms_norm_rounding_order_matches_reference_cpu_path_bf16():
    """manual_rms_norm rounds x * rsqrt(var) to bf16 and then gamma * that to
    bf16 again; the oracle must reproduce those two roundings bit for bit."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(64, 256, generator=g).to(torch.bfloat16)
    w = (1 + 0.02 * torch.randn(256, generator=g)).to(torch.bfloat16)
    ref = tp.rms_norm(x, w, 1e-5)
    assert ref.dtype == torch.bfloat16
    oy, _ = cf.rms_norm_fwd(x.double().numpy(), w.double().numpy(), 1e-5, out="bf16")
    same = np.mean(oy == ref.float().numpy())
    # torch evaluates x * rsqrt(var) in fp32, the oracle in fp64: a handful of
    # values that sit on a bf16 tie may differ
    assert same > 0.9995, same
    single = cf.round_to(
        w.double().numpy() * (x.double().numpy() * cf.rms_norm_fwd(x.double().numpy(), None, 1e-5)[1][:, None]),
        "bf16",
    )
    assert np.mean(single == ref.float().numpy()) < 0.99  # single rounding is measurably different


def test_layer_norm_single_rounding_matches_torch_cpu_bf16():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(64, 512, generator=g).to(torch.bfloat16)
    w = (1 + 0.02 * torch.randn(512, generator=g)).to(torch.bfloat16)
    b = (0.02 * torch.randn(512, generator=g)).to(torch.bfloat16)
    ref = tp.layer_norm(x, w, b, 1e-5)
    oy, _, _ = cf.layer_norm_fwd(x.double().numpy(), w.double().numpy(), b.double().numpy(), 1e-5, out="bf16")
    assert np.mean(oy == ref.float().numpy()) > 0.999


# ---------------------------------------------------------------- bias-GeLU
def test_bias_gelu_vs_torch_tanh_gelu_fp64():
    r = rng(40)
    x = torch.from_numpy(r.standard_normal((7, 24)) * 3).requires_grad_()
    b = torch.from_numpy(0.2 * r.standard_normal(24)).requires_grad_()
    g = torch.from_numpy(r.standard_normal((7, 24)))
    y = F.gelu(x + b, approximate="tanh")
    y.backward(g)
    oy = cf.bias_gelu_fwd(x.detach().numpy(), b.detach().numpy())
    # 0.79788456 is sqrt(2/pi) to fp32 precision: agreement to ~1e-8, not 1e-16
    assert np.allclose(oy, y.detach().numpy(), rtol=2e-7, atol=1e-8)
    dx, db = cf.bias_gelu_bwd(g.numpy(), x.detach().numpy(), b.detach().numpy())
    assert np.allclose(dx, x.grad.numpy(), rtol=2e-6, atol=1e-7)
    assert np.allclose(db, b.grad.numpy(), rtol=2e-6, atol=1e-6)
    # the explicit derivative of the reference equals autograd of its forward
    x2 = x.detach().clone().requires_grad_()
    tp.bias_gelu(x2, b.detach()).backward(g)
    assert np.allclose(dx, x2.grad.numpy(), rtol=1e-7, atol=1e-9)
    assert np.allclose(tp.bias_gelu_grad(g, x.detach(), b.detach()).numpy(), dx, rtol=1e-12, atol=1e-14)


def test_gelu_special_values():
    u = np.array([0.0, 1.5, -1.5, 30.0, -30.0])
    y = cf.bias_gelu_fwd(u, None)
    assert y[0] == 0
    assert np.isclose(y[1] - y[2], 1.5, rtol=1e-14)  # gelu(u) - gelu(-u) = u
    assert y[3] == 30.0 and abs(y[4]) == 0.0
    d, _ = cf.bias_gelu_bwd(np.ones(5), u, None)
    assert d[0] == 0.5 and d[3] == 1.0 and abs(d[4]) == 0.0
    eps = 1e-6
    fd = (cf.bias_gelu_fwd(u + eps, None) - cf.bias_gelu_fwd(u - eps, None)) / (2 * eps)
    assert np.allclose(d, fd, atol=1e-8)


def test_constants():
    assert np.float32(cf.GELU_A) == np.float32(np.sqrt(2 / np.pi))
    assert np.isclose(cf.GELU_C, 3 * cf.GELU_B * cf.GELU_A, rtol=1e-9)


# ---------------------------------------------------------------- bias-dropout-add
def test_bias_dropout_add_identity_and_scaling():
    r = rng(50)
    x, res = r.standard_normal((6, 16)), r.standard_normal((6, 16))
    b = r.standard_normal(16)
    out = cf.bias_dropout_add_fwd(x, b, res, None, 0.0)
    assert np.array_equal(out, x + b + res)
    keep = r.random((6, 16)) > 0.3
    out = cf.bias_dropout_add_fwd(x, b, None, keep, 0.3)
    scale = float(np.float32(1) / (np.float32(1) - np.float32(0.3)))
    assert np.array_equal(out[~keep], np.zeros((~keep).sum()))
    assert np.allclose(out[keep], ((x + b) * scale)[keep], rtol=1e-15)
    ref = tp.bias_dropout_add(torch.from_numpy(x), torch.from_numpy(b), torch.from_numpy(res), 0.3, True,
                              keep=torch.from_numpy(keep))
    assert np.allclose(cf.bias_dropout_add_fwd(x, b, res, keep, 0.3), ref.numpy(), rtol=3e-7, atol=3e-7)


def test_share_of_bf16_results_an_fp32_evaluation_rounds_the_other_way():
    """Where the 99.8 % of the 16-bit parity bar comes from: the same formula
    evaluated in float32 (every product and sum rounded, as a kernel does) and
    in float64, both then rounded to bfloat16, differ in one to three results
    in a thousand for bfloat16 operands with a dropout scale that is no power
    of two -- sums of short operands land next to rounding ties often -- and
    in none for p = 0.5, whose scale is exact."""
    r = rng(52)
    rows, cols = 64, 4096
    x = cf.round_to(r.standard_normal((rows, cols)), "bf16")
    res = cf.round_to(r.standard_normal((rows, cols)), "bf16")
    keep = np.ones((rows, cols), dtype=bool)
    for bias_std, p, low, high in ((0.02, 0.1, 5e-4, 2e-3), (0.1, 0.1, 1e-3, 4e-3), (0.1, 0.5, 0.0, 0.0)):
        b = cf.round_to(bias_std * r.standard_normal(cols), "bf16")
        exact = cf.bias_dropout_add_fwd(x, b, res, keep, p, out="bf16")
        single = cf.bias_dropout_add_fwd(x, b, res, keep, p, out="bf16", acc=np.float32)
        share = float(np.mean(exact != single))
        assert low <= share <= high, (bias_std, p, share)
        # one step of bfloat16 at most (sums that cancel carry float32's absolute error instead)
        assert np.all(np.abs(exact - single) <= np.maximum(2.0 ** -7 * np.abs(exact), 1e-6))


def test_bias_dropout_add_bwd_vs_autograd():
    r = rng(51)
    x = torch.from_numpy(r.standard_normal((5, 8))).requires_grad_()
    b = torch.from_numpy(r.standard_normal(8)).requires_grad_()
    res = torch.from_numpy(r.standard_normal((5, 8))).requires_grad_()
    keep = torch.from_numpy(r.random((5, 8)) > 0.25)
    g = torch.from_numpy(r.standard_normal((5, 8)))
    tp.bias_dropout_add(x, b, res, 0.25, True, keep=keep).backward(g)
    dx, db = cf.bias_dropout_add_bwd(g.numpy(), keep.numpy(), 0.25)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-7)
    assert np.allclose(db, b.grad.numpy(), rtol=1e-7)
    assert np.array_equal(res.grad.numpy(), g.numpy())


def test_autograd_sums_full_size_bias_grad():
    """The reference returns a [rows, cols] gradient for the [cols] bias
    (functional.py:84); autograd reduces it to the column sum."""

    class Fn(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, b):
            return x + b

        @staticmethod
        def backward(ctx, g):
            return g, g

    x = torch.randn(5, 3, dtype=torch.float64, requires_grad=True)
    b = torch.randn(3, dtype=torch.float64, requires_grad=True)
    g = torch.randn(5, 3, dtype=torch.float64)
    Fn.apply(x, b).backward(g)
    assert torch.allclose(b.grad, g.sum(0))


# ------------------------------------------------------- softmax + dropout
def test_softmax_dropout_vs_autograd_of_the_unfused_chain():
    """softmax -> dropout as the models chain them (modeling_gpt2.py:138-142):
    forward and backward of the oracle against torch autograd through
    softmax(where(hidden, -1e4, scale * x)) * keep / (1 - p) in float64, with an
    explicit keep mask; a wrong scale placement or a missing keep factor in the
    backward fails here."""
    r = np.random.default_rng(11)
    b, sq, sk, scale, p = 3, 5, 24, 0.37, 0.25
    x = torch.from_numpy(r.standard_normal((b, sq, sk))).requires_grad_(True)
    g = torch.from_numpy(r.standard_normal((b, sq, sk)))
    keep = r.random((b, sq, sk)) >= p
    hidden = cf.causal_hidden(sq, sk)
    t = torch.where(torch.from_numpy(hidden), torch.tensor(-1e4, dtype=torch.float64), x * scale)
    out = torch.softmax(t, -1) * torch.from_numpy(keep) / (1.0 - p)
    out.backward(g)
    o = cf.softmax_dropout_fwd(x.detach().numpy(), hidden, scale, keep, p)
    # the oracle's dropout scale is the float32 quotient 1 / (1 - p), as in the kernel
    assert np.allclose(o, out.detach().numpy(), rtol=1e-7, atol=1e-300)
    dx = cf.softmax_dropout_bwd(g.numpy(), x.detach().numpy(), hidden, scale, keep, p)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-6, atol=1e-12)
    # p = 0 / no mask: the plain softmax pair
    assert np.array_equal(
        cf.softmax_dropout_fwd(x.detach().numpy(), hidden, scale, None, 0.0),
        cf.softmax_causal_fwd(x.detach().numpy(), scale),
    )
    y = cf.softmax_causal_fwd(x.detach().numpy(), scale)
    assert np.allclose(
        cf.softmax_dropout_bwd(g.numpy(), x.detach().numpy(), hidden, scale, None, 0.0),
        cf.softmax_bwd(g.numpy(), y, scale), rtol=1e-13, atol=1e-300,
    )
    # dropped positions still receive a gradient through the normaliser
    assert (dx[~keep & ~np.broadcast_to(hidden, keep.shape)] != 0).any()


# ------------------------------------------- bias-dropout-add fused into a norm
@pytest.mark.parametrize("rms", [False, True])
def test_bias_dropout_add_norm_vs_autograd_of_the_unfused_chain(rms):
    """norm(keep * (x + b) / (1 - p) + residual) with an explicit keep mask and a
    second consumer of h (its gradient is dh_extra): forward and every gradient
    of the oracle against torch autograd in float64."""
    r = np.random.default_rng(5)
    n1, n2, p, eps = 7, 24, 0.2, 1e-5
    # the reference's RMS formula takes the variance in float32 even for float64 input
    rt = 2e-6 if rms else 1e-9
    x = torch.from_numpy(r.standard_normal((n1, n2))).requires_grad_(True)
    b = torch.from_numpy(r.standard_normal(n2)).requires_grad_(True)
    res = torch.from_numpy(r.standard_normal((n1, n2))).requires_grad_(True)
    gam = torch.from_numpy(1 + 0.1 * r.standard_normal(n2)).requires_grad_(True)
    bet = torch.from_numpy(0.1 * r.standard_normal(n2)).requires_grad_(True)
    keep = r.random((n1, n2)) >= p
    gy = torch.from_numpy(r.standard_normal((n1, n2)))
    gh = torch.from_numpy(r.standard_normal((n1, n2)))
    scale = float(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))
    h = (x + b) * torch.from_numpy(keep) * scale + res
    if rms:
        y = tp.rms_norm(h, gam, eps)
    else:
        y = torch.nn.functional.layer_norm(h, (n2,), gam, bet, eps)
    (y * gy).sum().backward(retain_graph=True)
    (h * gh).sum().backward()
    oy, oh, om, oi = cf.bias_dropout_add_norm_fwd(
        x.detach().numpy(), b.detach().numpy(), res.detach().numpy(), keep, p,
        gam.detach().numpy(), bet.detach().numpy(), eps, rms)
    assert np.allclose(oh, h.detach().numpy(), rtol=1e-13, atol=1e-300)
    assert np.allclose(oy, y.detach().numpy(), rtol=rt * 1e-2 if not rms else rt, atol=1e-13)
    dres, dx, dg, dbt, dbias = cf.bias_dropout_add_norm_bwd(
        gy.numpy(), gh.numpy(), oh, om, oi, gam.detach().numpy(), keep, p, rms)
    assert np.allclose(dres, res.grad.numpy(), rtol=rt, atol=1e-12 if not rms else 1e-6)
    assert np.allclose(dx, x.grad.numpy(), rtol=rt, atol=1e-12 if not rms else 1e-6)
    assert np.allclose(dbias, b.grad.numpy(), rtol=rt, atol=1e-12 if not rms else 1e-6)
    assert np.allclose(dg, gam.grad.numpy(), rtol=rt, atol=1e-12 if not rms else 1e-6)
    if not rms:
        assert np.allclose(dbt, bet.grad.numpy(), rtol=rt, atol=1e-12 if not rms else 1e-6)
    # without the second consumer the residual gradient is the plain norm backward
    d0 = cf.bias_dropout_add_norm_bwd(gy.numpy(), None, oh, om, oi, gam.detach().numpy(), None, 0.0, rms)
    plain = (cf.rms_norm_bwd(gy.numpy(), oh, oi, gam.detach().numpy())[0] if rms
             else cf.layer_norm_bwd(gy.numpy(), oh, om, oi, gam.detach().numpy())[0])
    assert np.array_equal(d0[0], plain) and np.array_equal(d0[1], plain)
