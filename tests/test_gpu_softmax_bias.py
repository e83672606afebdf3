"""Softmax of scores with an additive floating-point term, y = softmax(scale * x + M),
forward and backward, with and without the fused dropout, on the GPU through the
C ABI.  This is the form in which the reference's models mask and bias their
scores: the -10000 mask of oslo/transformers/models/bert/modeling_bert.py:298-306
and models/gpt2/modeling_gpt2.py:136, 573-581, the finfo.min mask of
models/bart/modeling_bart.py:123-136, 262-284, the relative-position bias of
models/t5/modeling_t5.py:508-514.

Oracle: oracle/closed_form.py softmax_bias_fwd (float64, the sum rounded to
float32 once, as the kernel's multiply-add forms it), pinned against
torch.softmax(scale * x + M) and autograd in tests/test_oracle_closed_form.py.
Tolerances: float32 1e-5 relative, 16-bit <= 1 ulp of the once-rounded oracle
(helpers.check); zeros of hidden keys and dropout keep bits are exact."""
import numpy as np
import pytest
import torch

from helpers import check, f64, randn
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16


def lowest(dtype):
    return float(torch.finfo(dtype).min)


def make_bias(kind, b, np_, sq, sk, dtype, seed):
    """The additive term of one of the reference's call sites, as a CPU tensor."""
    r = np.random.default_rng(seed)
    if kind in ("m10000", "min", "inf", "min32"):
        # key-padding mask [b, 1, 1, sk]: 0 for visible keys; sample 0 sees every key
        valid = r.integers(max(1, sk // 4), sk + 1, size=b)
        valid[0] = sk
        pad = torch.from_numpy(np.arange(sk)[None, :] >= valid[:, None]).view(b, 1, 1, sk)
        fill = {"m10000": -10000.0, "min": lowest(dtype), "inf": float("-inf"),
                "min32": lowest(F32)}[kind]
        m = torch.zeros(b, 1, 1, sk, dtype=F32).masked_fill(pad, fill)
        return m.to(F32 if kind == "min32" else dtype)
    if kind == "t5":        # position bias shared by the batch
        return randn((1, np_, sq, sk), dtype, seed=seed, std=2.0)
    if kind == "t5_f32":    # ... in float32 next to 16-bit scores (autocast)
        return randn((1, np_, sq, sk), F32, seed=seed, std=2.0)
    if kind == "full":
        return randn((b, np_, sq, sk), dtype, seed=seed, std=2.0)
    if kind == "perq":      # [b, 1, sq, sk]: HF's 4-D mask, finfo.min above a random staircase
        m = torch.zeros(b, 1, sq, sk, dtype=F32)
        cut = torch.from_numpy(r.integers(1, sk + 1, size=(b, 1, sq, 1)))
        m = m.masked_fill(torch.arange(sk).view(1, 1, 1, sk) >= cut, lowest(dtype))
        return m.to(dtype)
    if kind == "alibi":     # [1, np, 1, sk] slopes * key position
        slopes = torch.tensor([2.0 ** -(i + 1) for i in range(np_)]).view(1, np_, 1, 1)
        return (slopes * -torch.arange(sk, dtype=F32).view(1, 1, 1, sk).flip(-1)).to(dtype)
    raise ValueError(kind)


CASES = [
    # (b, np, sq, sk, dtype, scale, kind, causal)
    (3, 2, 64, 128, BF16, 0.125, "m10000", False),
    (3, 2, 64, 128, F16, 0.125, "m10000", False),
    (2, 2, 32, 512, F32, 0.125, "m10000", False),
    (3, 2, 64, 1024, F16, 0.125, "min", False),        # configuration-3 row length
    (3, 2, 64, 1024, BF16, 0.125, "min", False),
    (3, 2, 16, 2048, BF16, 0.10206207, "inf", False),
    (2, 2, 32, 512, F32, 0.125, "min", False),
    (2, 2, 32, 512, BF16, 0.125, "min32", False),      # float32 term, 16-bit scores
    (2, 4, 128, 128, BF16, 1.0, "t5", False),
    (2, 4, 128, 128, F16, 1.0, "t5_f32", False),
    (2, 3, 96, 96, F32, 1.0, "t5", False),             # three chunks per lane
    (2, 2, 48, 256, BF16, 0.25, "full", False),
    (2, 2, 48, 256, F16, 0.25, "perq", False),
    (2, 4, 40, 320, BF16, 0.125, "alibi", True),
    (3, 2, 128, 128, BF16, 0.125, "m10000", True),     # GPT-2: causal + additive padding mask
    (2, 2, 512, 512, F32, 0.125, "min", True),
    (2, 2, 256, 2048, BF16, 0.10206207, "min", True),  # sq != sk with the diagonal
    (2, 2, 37, 64, F16, 0.5, "inf", True),
    (2, 2, 64, 40, BF16, 0.5, "t5", True),             # sq > sk: the diagonal hides whole rows
    # the same where rows lie side by side in a wave: a row without any key next to rows that see keys
    (2, 2, 37, 20, F32, 0.5, "t5", True),
    (2, 2, 40, 64, BF16, 0.5, "perq", True),
    (2, 3, 70, 128, F16, 0.25, "m10000", True),
    (2, 1, 300, 256, BF16, 0.25, "t5", True),
    (1, 2, 600, 512, BF16, 0.25, "min", True),         # and with a wave per row
    (1, 1, 2060, 2052, F16, 0.25, "t5", True),         # one workgroup per row
    (1, 2, 8, 4096, BF16, 1.0, "min", False),          # two waves per row
    (2, 1, 4, 16384, F16, 1.0, "t5", False),
    (2, 2, 33, 33, F32, 0.7, "m10000", False),         # odd length: scalar kernels
    (2, 2, 50, 50, BF16, 0.5, "t5", True),
    (2, 2, 20, 1004, BF16, 0.25, "min", False),
    (2, 1, 5, 2051, BF16, 0.25, "t5_f32", False),      # one workgroup per row
    (2, 2, 100, 768, F16, 0.125, "perq", False),
    (3, 1, 1, 8, F32, 2.0, "m10000", False),
    (2, 2, 7, 16, BF16, 1.0, "full", True),
    (4, 3, 9, 64, F16, 0.5, "alibi", False),
]


def run_pair(k, x, dy, bias, scale, causal, device, skip):
    y = k.softmax_bias_forward(x.to(device), bias.to(device), scale, causal=causal, skip_hidden=skip)
    dx = k.softmax_bias_backward(dy.to(device), y, scale, bias=bias.to(device), causal=causal,
                                 skip_hidden=skip)
    return y, dx


@pytest.mark.parametrize("b,np_,sq,sk,dtype,scale,kind,causal", CASES)
def test_bias_softmax(device, b, np_, sq, sk, dtype, scale, kind, causal, rows_per_wave=(1, 0)):
    # rows_per_wave: the override both launches below run under, and the value put back afterwards
    x = randn((b, np_, sq, sk), dtype, seed=sq + sk, std=2.0)
    dy = randn((b, np_, sq, sk), dtype, seed=sq + sk + 1)
    bias = make_bias(kind, b, np_, sq, sk, dtype, seed=sk)
    k = _C.get_softmax_kernel()
    oy = cf.softmax_bias_fwd(f64(x), f64(bias), scale, causal=causal)
    finite_rows = np.isfinite(oy).all(-1)
    if causal and sq > sk:
        # the diagonal hides every key of the first sq - sk queries (a -inf triangle
        # added to the scores gives NaN in torch): the kernels write zeros there
        assert not finite_rows[..., : sq - sk].any() and finite_rows[..., sq - sk:].all()
    else:
        assert finite_rows.all()
    results = []
    for skip in (False, True):
        # (the same launch shape for both: two builds of a kernel may round a 16-bit
        #  output once or twice, which differs on ties)
        _C.tune("softmax_rows_per_wave", rows_per_wave[0])
        try:
            y, dx = run_pair(k, x, dy, bias, scale, causal, device, skip)
        finally:
            _C.tune("softmax_rows_per_wave", rows_per_wave[1])
        ycpu = y.cpu()
        fr = torch.from_numpy(finite_rows)
        assert (ycpu[~fr] == 0).all() and (dx.cpu()[~fr] == 0).all()
        check(ycpu[fr], oy[finite_rows], "bias softmax fwd (skip=%s)" % skip, atol=1e-9)
        # a key whose probability underflows in the oracle is an exact zero here too
        # wherever its term hides it (-inf, the lowest value, -10000 next to a visible key)
        hidden = np.broadcast_to(f64(bias) <= -10000.0, oy.shape) & finite_rows[..., None]
        if causal:
            hidden = hidden | (cf.causal_hidden(sq, sk) & finite_rows[..., None])
        assert (ycpu[torch.from_numpy(hidden & (oy == 0))] == 0).all()
        odx = cf.softmax_bwd(f64(dy)[finite_rows], f64(ycpu)[finite_rows], scale)
        check(dx.cpu()[fr], odx, "bias softmax bwd (skip=%s)" % skip, atol=1e-7)
        results.append((ycpu, dx.cpu()))
    # leaving hidden logits unread changes no bit
    assert torch.equal(results[0][0][fr], results[1][0][fr])
    assert torch.equal(results[0][1][fr], results[1][1][fr])
    # the backward pass without the term is the same function
    dx0 = k.softmax_bias_backward(dy.to(device), results[0][0].to(device), scale, causal=causal)
    assert torch.equal(dx0.cpu()[fr], results[0][1][fr])
    gi = dy.to(device).clone()
    ri = k.softmax_bias_backward(gi, results[0][0].to(device), scale, bias=bias.to(device),
                                 causal=causal, inplace=True)
    assert ri.data_ptr() == gi.data_ptr() and torch.equal(ri.cpu()[fr], results[0][1][fr])


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_padding_term_equals_the_boolean_mask_kernel(device, dtype):
    """With a visible key in every row, the additive -10000 / lowest / -inf key
    mask gives the probabilities of the boolean-mask kernel, zeros included."""
    b, np_, sq, sk = 3, 2, 40, 256
    x = randn((b, np_, sq, sk), dtype, seed=5, std=2.0)
    k = _C.get_softmax_kernel()
    for kind in ("m10000", "min", "inf"):
        bias = make_bias(kind, b, np_, sq, sk, dtype, seed=9)
        pad = (bias != 0)
        y = k.softmax_bias_forward(x.to(device), bias.to(device), 0.125).cpu()
        yb = k.fused_scaled_masked_softmax_forward(x.to(device), pad.to(device), 0.125).cpu()
        # the boolean kernel keeps its logits in the log2 domain, this one in the natural
        # domain: the same function to an ulp of float32 before the output rounding
        d = (y.float() - yb.float()).abs()
        assert float(d.max()) <= (2e-7 if dtype == F32 else float(torch.finfo(dtype).eps))
        assert torch.equal(y == 0, yb == 0)


def test_rows_without_a_visible_key(device):
    """-10000 everywhere: softmax(scale * x), which is what
    modeling_bert.py:298-306 computes for such a row; the lowest float
    everywhere: uniform (the term absorbs the logit); -inf everywhere: NaN, as
    torch.softmax returns; a mixture of -inf and the lowest float: uniform
    over the finite ones.  With and without skipping."""
    b, np_, sq, sk = 2, 2, 4, 64
    x = randn((b, np_, sq, sk), F32, seed=1, std=2.0)
    dy = randn((b, np_, sq, sk), F32, seed=2)
    k = _C.get_softmax_kernel()
    for skip in (False, True):
        for fill, dtype in ((-10000.0, F32), (lowest(F32), F32), (lowest(BF16), BF16),
                            (float("-inf"), F32), (lowest(F16), F16), (-10000.0, BF16)):
            xx, gg = x.to(dtype), dy.to(dtype)
            bias = torch.zeros(b, 1, 1, sk, dtype=dtype)
            bias[1] = fill  # sample 1 sees nothing
            y, dx = run_pair(k, xx, gg, bias, 0.5, False, device, skip)
            y, dx = y.cpu(), dx.cpu()
            oy = cf.softmax_bias_fwd(f64(xx), f64(bias), 0.5)
            if fill == float("-inf"):
                assert torch.isnan(y[1]).all() and np.isnan(oy[1]).all()
                assert torch.isnan(dx[1]).all()
                check(y[0], oy[0], "visible sample", atol=1e-9)
                continue
            check(y, oy, "row without a visible key, fill %g" % fill, atol=1e-9)
            if fill < -1e38:
                assert (y[1] == 1.0 / sk).all()
            else:
                assert not torch.allclose(y[1].float(), torch.full_like(y[1].float(), 1.0 / sk), rtol=0.05)
            check(dx, cf.softmax_bwd(f64(gg), f64(y), 0.5), "its backward", atol=1e-7)
        bias = torch.full((b, 1, 1, sk), lowest(F32))
        bias[..., ::2] = float("-inf")
        y = k.softmax_bias_forward(x.to(device), bias.to(device), 0.5, skip_hidden=skip).cpu()
        assert (y[..., 1::2] == 2.0 / sk).all() and (y[..., ::2] == 0).all()


def test_term_layouts(device):
    """Expanded views (stride 0), fewer than four dimensions, a term whose
    rows are not 16-byte aligned (scalar kernels), a term in another float
    type (converted to float32 by the binding)."""
    b, np_, sq, sk = 2, 3, 16, 64
    x = randn((b, np_, sq, sk), BF16, seed=3, std=2.0)
    k = _C.get_softmax_kernel()
    base = randn((np_, sq, sk), BF16, seed=4, std=2.0)
    want = cf.softmax_bias_fwd(f64(x), f64(base)[None], 0.3)
    for bias in (base, base[None], base[None].expand(b, np_, sq, sk), base.to(F16),
                 base.double()):
        y = k.softmax_bias_forward(x.to(device), bias.to(device), 0.3)
        check(y, want, "layout %s %s" % (list(bias.shape), bias.dtype), atol=1e-9)
    # rows of the term 2 * 68 bytes apart: not vectorisable
    wide = randn((sq, sk + 4), BF16, seed=5, std=2.0)
    view = wide[:, 2:sk + 2]
    want = cf.softmax_bias_fwd(f64(x), f64(view)[None, None], 0.3)
    y = k.softmax_bias_forward(x.to(device), wide.to(device)[:, 2:sk + 2], 0.3)
    check(y, want, "unaligned term", atol=1e-9)
    # a per-key vector [sk] and a column [sq, 1] (constant per row: changes nothing)
    vec = randn((sk,), BF16, seed=6, std=2.0)
    check(k.softmax_bias_forward(x.to(device), vec.to(device), 0.3),
          cf.softmax_bias_fwd(f64(x), f64(vec), 0.3), "vector term", atol=1e-9)
    col = randn((sq, 1), BF16, seed=7, std=2.0)
    check(k.softmax_bias_forward(x.to(device), col.to(device), 0.3),
          cf.softmax_bias_fwd(f64(x), f64(col), 0.3), "column term", atol=1e-9)
    with pytest.raises(RuntimeError):
        k.softmax_bias_forward(x.to(device), randn((b, np_, sq, sk + 1), BF16, 1).to(device), 0.3)
    with pytest.raises(RuntimeError):
        k.softmax_bias_forward(x.to(device), torch.zeros(b, np_, sq, sk, dtype=torch.bool, device=device), 0.3)
    with pytest.raises(RuntimeError):
        k.softmax_bias_forward(x.to(device), base, 0.3)  # term on the CPU


DROPOUT_CASES = [
    (2, 2, 64, 128, BF16, 0.125, "m10000", False, 0.1),
    (2, 2, 32, 512, F32, 0.125, "min", False, 0.1),
    (2, 2, 64, 1024, F16, 0.125, "min", True, 0.1),
    (2, 4, 128, 128, BF16, 1.0, "t5", False, 0.1),
    (2, 4, 96, 96, F16, 1.0, "t5_f32", False, 0.2),
    (2, 2, 16, 2048, BF16, 0.10206207, "inf", True, 0.1),
    (2, 2, 33, 33, F32, 0.7, "full", False, 0.1),
    (2, 1, 5, 2051, BF16, 0.25, "t5", False, 0.1),
    (2, 2, 20, 1004, F16, 0.25, "perq", False, 0.1),
    (1, 2, 8, 4096, BF16, 1.0, "min", False, 0.1),
    # sq > sk under the diagonal: rows without any key, side by side with rows that see keys and alone in a wave
    (2, 2, 37, 20, F32, 0.5, "perq", True, 0.1),
    (2, 2, 40, 64, BF16, 0.5, "t5", True, 0.1),
    (2, 2, 300, 256, F16, 0.25, "min", True, 0.1),
    (1, 2, 600, 512, BF16, 0.25, "t5", True, 0.1),
    (2, 2, 50, 44, BF16, 0.5, "t5", True, 0.1),        # one wave per row, scalar accesses
    (1, 1, 2060, 2052, F16, 0.25, "min", True, 0.1),   # one workgroup per row
]


@pytest.mark.parametrize("b,np_,sq,sk,dtype,scale,kind,causal,p", DROPOUT_CASES)
def test_bias_softmax_dropout(device, b, np_, sq, sk, dtype, scale, kind, causal, p):
    seed, offset = 91 + sk, 4 * sq
    x = randn((b, np_, sq, sk), dtype, seed=sq + sk, std=2.0)
    g = randn((b, np_, sq, sk), dtype, seed=sq + sk + 1)
    bias = make_bias(kind, b, np_, sq, sk, dtype, seed=sk)
    k = _C.get_softmax_kernel()
    n = b * np_ * sq * sk
    keep = philox.keep_mask(n, p, seed, offset).reshape(b, np_, sq, sk).astype(bool)
    oo = cf.softmax_bias_dropout_fwd(f64(x), f64(bias), scale, keep, p, causal=causal)
    odx = cf.softmax_bias_dropout_bwd(f64(g), f64(x), f64(bias), scale, keep, p, causal=causal)
    plain = k.softmax_bias_forward(x.to(device), bias.to(device), scale, causal=causal).cpu()
    # queries that the diagonal leaves without any key (sq > sk; NaN in the oracle as in torch): zeros here
    fr = np.isfinite(oo).all(-1)
    assert fr.all() or (causal and sq > sk and not fr[..., : sq - sk].any() and fr[..., sq - sk:].all())
    frt = torch.from_numpy(fr)
    outs = []
    for skip in (False, True):
        out, stats = k.softmax_bias_dropout_forward(x.to(device), bias.to(device), scale, p, seed,
                                                    offset, causal=causal, skip_hidden=skip)
        plain = k.softmax_bias_forward(x.to(device), bias.to(device), scale, causal=causal,
                                       skip_hidden=skip).cpu()
        assert (out.cpu()[~frt] == 0).all() and torch.isfinite(stats).all()
        check(out.cpu()[frt], oo[fr], "bias softmax dropout fwd", atol=1e-9)
        ocpu = out.cpu()
        # the keep decisions are the Philox stream over the flattened output, bit for bit
        assert (ocpu[torch.from_numpy(~keep)] == 0).all(), "dropped elements must be exactly 0"
        assert (ocpu[torch.from_numpy(keep) & (plain != 0)] != 0).all(), "kept elements must survive"
        dx = k.softmax_bias_dropout_backward(g.to(device), x.to(device), bias.to(device), stats, scale,
                                             p, seed, offset, causal=causal, skip_hidden=skip)
        assert (dx.cpu()[~frt] == 0).all()
        check(dx.cpu()[frt], odx[fr], "bias softmax dropout bwd", atol=2e-7)
        outs.append((ocpu, dx.cpu()))
        # p = 0 reproduces the plain kernel bit for bit
        out0, _ = k.softmax_bias_dropout_forward(x.to(device), bias.to(device), scale, 0.0, seed,
                                                 offset, causal=causal, skip_hidden=skip)
        assert torch.equal(out0.cpu(), plain)
    # (the two launch shapes may round a 16-bit output once or twice: equal up to ties)
    assert float((outs[0][0].float() - outs[1][0].float()).abs().max()) <= float(torch.finfo(dtype).eps)


def test_dropout_row_without_a_visible_key(device):
    """The statistics of a row whose maximum is a hiding term: backward must
    read such a row in full."""
    b, np_, sq, sk = 2, 2, 8, 128
    x = randn((b, np_, sq, sk), BF16, seed=1, std=2.0)
    g = randn((b, np_, sq, sk), BF16, seed=2)
    bias = torch.zeros(b, 1, 1, sk, dtype=BF16)
    bias[1] = lowest(BF16)
    bias[0, ..., sk // 2:] = lowest(BF16)
    p, seed, offset = 0.25, 5, 8
    keep = philox.keep_mask(b * np_ * sq * sk, p, seed, offset).reshape(b, np_, sq, sk).astype(bool)
    k = _C.get_softmax_kernel()
    for skip in (False, True):
        out, stats = k.softmax_bias_dropout_forward(x.to(device), bias.to(device), 0.5, p, seed, offset,
                                                    skip_hidden=skip)
        check(out, cf.softmax_bias_dropout_fwd(f64(x), f64(bias), 0.5, keep, p), "fwd", atol=1e-9)
        dx = k.softmax_bias_dropout_backward(g.to(device), x.to(device), bias.to(device), stats, 0.5, p,
                                             seed, offset, skip_hidden=skip)
        check(dx, cf.softmax_bias_dropout_bwd(f64(g), f64(x), f64(bias), 0.5, keep, p), "bwd", atol=2e-7)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("scale", [1.0, 0.25])
def test_autograd_with_a_learned_term(device, dtype, scale):
    """scaled_bias_softmax(+ dropout) against torch autograd of the unfused
    chain in float64: gradient of the scores and of a term that requires one
    (T5's relative-attention bias: summed over the batch it is broadcast along)."""
    import oslo_amd.torch.nn as onn

    b, np_, sq, sk = 3, 4, 32, 64
    x = randn((b, np_, sq, sk), dtype, seed=1, std=2.0)
    m = randn((1, np_, sq, sk), dtype, seed=2, std=1.5)
    g = randn((b, np_, sq, sk), dtype, seed=3)
    xd, md = x.to(device).requires_grad_(), m.to(device).requires_grad_()
    y = onn.scaled_bias_softmax(xd, md, scale)
    y.backward(g.to(device))
    xr, mr = x.double().requires_grad_(), m.double().requires_grad_()
    ref = torch.softmax(scale * xr + mr, dim=-1)
    ref.backward(g.double())
    check(y, ref.detach().numpy(), "fwd", atol=1e-9)
    tol = dict(rtol=1e-4, atol=1e-6) if dtype == F32 else dict(rtol=3e-2, atol=2e-3)
    assert torch.allclose(xd.grad.cpu().double(), xr.grad, **tol)
    assert md.grad.shape == md.shape and md.grad.dtype == dtype
    assert torch.allclose(md.grad.cpu().double(), mr.grad, **tol)
    # only the term asks for a gradient
    x2, m2 = x.to(device), m.to(device).requires_grad_()
    onn.scaled_bias_softmax(x2, m2, scale).backward(g.to(device))
    assert torch.equal(m2.grad, md.grad)
    # with dropout: the keep mask is recovered from the output (kept = non-zero)
    torch.manual_seed(7)
    xd2, md2 = x.to(device).requires_grad_(), m.to(device).requires_grad_()
    out = onn.scaled_bias_softmax_dropout(xd2, md2, scale, p=0.2, training=True)
    out.backward(g.to(device))
    keep = (out.detach().cpu() != 0).double()
    xr2, mr2 = x.double().requires_grad_(), m.double().requires_grad_()
    ps = float(np.float32(1.0) / (np.float32(1.0) - np.float32(0.2)))
    (torch.softmax(scale * xr2 + mr2, dim=-1) * keep * ps).backward(g.double())
    assert 0.7 < keep.mean().item() < 0.9
    assert torch.allclose(xd2.grad.cpu().double(), xr2.grad, **tol)
    assert torch.allclose(md2.grad.cpu().double(), mr2.grad, **tol)


def test_module_takes_additive_and_per_head_masks(device):
    """FusedScaleMaskSoftmax with the mask exactly as the reference's BERT and
    GPT-2 build it ((1 - m) * -10000, [b, 1, 1, sk]), with a T5-style bias,
    with a boolean mask per head, with and without the causal type: the fused
    branch against the module's own torch branch."""
    from oslo_amd.torch.nn.modules.softmax import AttnMaskType, FusedScaleMaskSoftmax

    b, np_, sq, sk = 2, 3, 48, 64
    x = randn((b, np_, sq, sk), F32, seed=2, std=2.0).to(device)
    valid = torch.tensor([sk, 40])
    attn = (torch.arange(sk)[None, :] < valid[:, None]).float()
    hf_mask = ((1.0 - attn) * -10000.0).view(b, 1, 1, sk).to(device)
    t5_bias = randn((1, np_, sq, sk), F32, seed=4, std=2.0).to(device)
    per_head = (torch.rand(b, np_, sq, sk, generator=torch.Generator().manual_seed(1)) < 0.3)
    per_head[..., 0] = False
    per_head = per_head.to(device)
    for mask_type in (AttnMaskType.padding, AttnMaskType.causal):
        fused = FusedScaleMaskSoftmax(attn_mask_type=mask_type, scale=0.25)
        unfused = FusedScaleMaskSoftmax(attn_mask_type=mask_type, scale=0.25,
                                        scaled_masked_softmax_fusion=False)
        for mask in (hf_mask, t5_bias, per_head, t5_bias[0], hf_mask.double()):
            assert fused.is_kernel_available(mask, b, np_, sq, sk, input=x)
            a, c = fused(x, mask), unfused(x, mask)
            assert torch.allclose(a, c, rtol=1e-5, atol=1e-7), (mask_type, mask.shape, mask.dtype)
    # the gradient reaches a learned term through the module
    bias = t5_bias.clone().requires_grad_()
    xg = x.clone().requires_grad_()
    FusedScaleMaskSoftmax(scale=0.25)(xg, bias).square().sum().backward()
    br, xr = t5_bias.clone().requires_grad_(), x.clone().requires_grad_()
    torch.softmax(0.25 * xr + br, -1).square().sum().backward()
    assert torch.allclose(bias.grad, br.grad, rtol=1e-4, atol=1e-6)
    assert torch.allclose(xg.grad, xr.grad, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("b,np_,sq,sk,dtype,causal", [
    (3, 4, 50, 256, BF16, False),     # 600 rows: workgroups not a multiple of 8, batch of 3
    (16, 2, 64, 1024, F16, False),    # two row sets ... one per workgroup, 2048 workgroups
    (5, 3, 7, 64, F32, True),         # rows side by side in a wave, few workgroups
    (2, 2, 33, 33, BF16, False),      # scalar kernels
    (4, 2, 8, 4096, BF16, True),      # two waves per row
])
def test_row_order_of_a_term_shared_by_the_batch(device, b, np_, sq, sk, dtype, causal):
    """A position bias [1, np, sq, sk]: the kernels visit the rows in runs of
    softmax_bias_group rows of one batch entry followed by the same rows of
    the next entry (softmax_bias_order 2, the default), also spread the
    workgroups so that one die works on consecutive rows (3), or keep the
    stored order (1).  The order changes no bit of any row."""
    x = randn((b, np_, sq, sk), dtype, seed=3, std=2.0)
    g = randn((b, np_, sq, sk), dtype, seed=4)
    bias = randn((1, np_, sq, sk), dtype, seed=5, std=2.0)
    k = _C.get_softmax_kernel()
    want = cf.softmax_bias_fwd(f64(x), f64(bias), 0.25, causal=causal)
    seed, offset, p = 11, 16, 0.2
    keep = philox.keep_mask(x.numel(), p, seed, offset).reshape(x.shape).astype(bool)
    outs = []
    for order, group in ((1, 0), (2, 0), (3, 0), (2, 1), (3, 1), (2, 8), (3, 64)):
        _C.tune("softmax_bias_order", order)
        _C.tune("softmax_bias_group", group)
        try:
            y = k.softmax_bias_forward(x.to(device), bias.to(device), 0.25, causal=causal)
            o, stats = k.softmax_bias_dropout_forward(x.to(device), bias.to(device), 0.25, p, seed, offset,
                                                      causal=causal)
            dx = k.softmax_bias_dropout_backward(g.to(device), x.to(device), bias.to(device), stats, 0.25, p,
                                                 seed, offset, causal=causal)
        finally:
            _C.tune("softmax_bias_order", 0)
            _C.tune("softmax_bias_group", 0)
        check(y, want, "order %d fwd" % order, atol=1e-9)
        check(o, cf.softmax_bias_dropout_fwd(f64(x), f64(bias), 0.25, keep, p, causal=causal),
              "order %d dropout fwd" % order, atol=1e-9)
        check(dx, cf.softmax_bias_dropout_bwd(f64(g), f64(x), f64(bias), 0.25, keep, p, causal=causal),
              "order %d dropout bwd" % order, atol=2e-7)
        outs.append((y.cpu(), o.cpu(), dx.cpu(), stats.cpu()))
    for other in outs[1:]:
        for a, c in zip(outs[0], other):
            assert torch.equal(a, c)
