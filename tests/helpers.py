"""Shared helpers of the test-suite: seeded inputs and the parity metrics.

Parity metrics (the tolerances the tests state):
  fp32 outputs   |a - t| <= 1e-5 * |t| + atol, t = float64 oracle, atol a small
                 multiple of the output scale for values that cancel to ~0.
  16-bit outputs (1) against the float64 oracle rounded once to the storage
                 type: at least 99.8 % of the elements bit-identical and no
                 element further than 1 ulp; (2) relative L2 error against the
                 unrounded float64 oracle <= 2e-3, or what the correctly
                 rounded oracle itself reaches where that is more (values that
                 crowd just above a power of two: up to 2.3e-3 in bf16).
                 (A per-element 2e-3 bound is not meaningful for bf16, whose
                 half-ulp is 3.9e-3: two correct roundings of values 1e-7
                 apart can differ by a full ulp.)
"""
import numpy as np
import torch

NP_NAME = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}


def randn(shape, dtype, seed, std=1.0, mean=0.0):
    """Seeded N(mean, std) drawn on the CPU in fp32, then cast to `dtype`."""
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(shape, generator=g, dtype=torch.float32) * std + mean
    return t.to(dtype)


def f64(t):
    """Exact values of a tensor as a float64 numpy array."""
    return t.detach().to("cpu").to(torch.float64).numpy()


def _ordered_int(t):
    if t.dtype == torch.float32:
        i = t.contiguous().view(torch.int32).to(torch.int64)
        mag = 0x7FFFFFFF
    else:
        i = t.contiguous().view(torch.int16).to(torch.int64)
        mag = 0x7FFF
    return torch.where(i >= 0, i, -(i & mag))


def ulp_distance(a, b):
    """Elementwise distance in units of the storage type's spacing."""
    assert a.dtype == b.dtype and a.shape == b.shape
    return (_ordered_int(a.cpu()) - _ordered_int(b.cpu())).abs()


def rel_l2(actual64, truth64):
    num = np.linalg.norm((actual64 - truth64).ravel())
    den = np.linalg.norm(truth64.ravel())
    return float(num / den) if den > 0 else float(num)


def check_lowp(actual, truth64, what, min_exact=0.998, max_ulp=1, l2_tol=2e-3, atol=0.0,
               single_rounding_too=False):
    """16-bit parity (see module docstring).  `actual` is a torch tensor of the
    storage dtype, `truth64` the float64 oracle (unrounded).  An element whose
    absolute error is within `atol` counts as exact: results that cancel to
    almost nothing carry the absolute error of the fp32 arithmetic, which can be
    many ulps of a tiny value.

    The expected value is the oracle rounded to float32 and then to the storage
    type, the two roundings of an fp32 evaluation.  `single_rounding_too` also
    accepts the oracle rounded to float16 directly: where the last operation is
    a multiply-add the hardware can form it and round it to float16 in one
    instruction, which differs from the two roundings exactly when the fp32
    value falls on a float16 tie -- common for 16-bit operands times short
    constants (0.9 m + 0.1 g)."""
    actual = actual.detach().cpu()
    truth64 = np.asarray(truth64, dtype=np.float64).reshape(actual.shape)
    expect = torch.from_numpy(truth64).to(torch.float32).to(actual.dtype)
    assert torch.isfinite(actual.float()).all(), what + ": non-finite output"
    d = ulp_distance(actual, expect)
    if single_rounding_too and actual.dtype == torch.float16:
        direct = torch.from_numpy(truth64.astype(np.float16))
        d = torch.minimum(d, ulp_distance(actual, direct))
    if atol > 0:
        within = torch.from_numpy(np.abs(f64(actual) - truth64) <= atol)
        d = torch.where(within, torch.zeros_like(d), d)
    exact = float((d == 0).double().mean()) if d.numel() else 1.0
    worst = int(d.max()) if d.numel() else 0
    l2 = rel_l2(f64(actual), truth64)
    # the L2 bound presumes enough elements to average over; a handful of
    # values can each sit at the half-ulp worst case (2^-9 for bf16)
    l2_bound = l2_tol if actual.numel() >= 256 else 2 * l2_tol
    # values that crowd just above a power of two (a near-uniform softmax row of
    # 1024 keys: every probability ~ 2^-10) carry the largest relative rounding
    # error of the storage type, 2.3e-3 rms in bf16: the bound is never tighter
    # than what the correctly rounded oracle itself achieves
    l2_bound = max(l2_bound, 1.02 * rel_l2(f64(expect), truth64))
    assert worst <= max_ulp, "%s: %d ulp off the rounded oracle (exact %.5f)" % (what, worst, exact)
    # a small tensor may hold a few values that sit on a rounding tie
    allowed = max(3.0, (1.0 - min_exact) * actual.numel()) if min_exact < 1.0 else 0.0
    mismatches = int((d != 0).sum()) if d.numel() else 0
    assert mismatches <= allowed, "%s: only %.5f bit-identical (%d elements differ)" % (what, exact, mismatches)
    # (a result that is within the absolute floor everywhere -- a gradient that cancels to
    # subnormal float16 values, say -- has no meaningful relative error)
    if not (atol > 0 and bool(np.all(np.abs(f64(actual) - truth64) <= atol))):
        assert l2 <= l2_bound, "%s: relative L2 error %.3e > %.1e" % (what, l2, l2_bound)
    return exact, worst, l2


def check_f32(actual, truth64, what, rtol=1e-5, atol=1e-6):
    a = f64(actual)
    t = np.asarray(truth64, dtype=np.float64).reshape(a.shape)
    assert np.isfinite(a).all(), what + ": non-finite output"
    err = np.abs(a - t)
    bound = rtol * np.abs(t) + atol
    bad = err > bound
    assert not bad.any(), "%s: %d elements off, worst |err| %.3e at |t| %.3e" % (
        what, int(bad.sum()), float(err[bad].max()), float(np.abs(t)[bad][err[bad].argmax()]))
    return float((err / (np.abs(t) + atol / rtol)).max())


def check(actual, truth64, what, atol=1e-6, **kw):
    """`atol` is the absolute floor for both kinds of output."""
    if actual.dtype == torch.float32:
        return check_f32(actual, truth64, what, atol=atol)
    return check_lowp(actual, truth64, what, atol=atol, **kw)
