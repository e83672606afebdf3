"""Committed vectors of the softmax with an additive floating-point term
(tests/golden/softmax_bias_vectors.npz, written by
tests/golden/make_fixtures_softmax_bias.py from torch's float64 evaluation of
the reference's unfused chains): the oracle must agree with them (CPU) and the
HIP kernels must match them through the C ABI (GPU)."""
import os

import numpy as np
import pytest
import torch

from helpers import check
from oracle import closed_form as cf
from oracle import philox

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "softmax_bias_vectors.npz")

# name -> (dtype of the scores, scale, causal)
CASES = {"gpt2": (torch.bfloat16, 0.125, True), "bart": (torch.float16, 0.25, False),
         "t5": (torch.float32, 1.0, False)}
DROP = dict(dtype=torch.bfloat16, scale=0.125, p=0.2, seed=31, offset=16)


@pytest.fixture(scope="module")
def vec():
    return {k: v.astype(np.float64) if v.dtype == np.float32 else v
            for k, v in np.load(PATH, allow_pickle=False).items()}


def test_oracle_agrees_with_the_committed_vectors(vec):
    """The oracle rounds scale * x + M to float32 once (as the kernel's multiply-add
    does), torch's float64 chain does not: equal to float32 resolution of the sum."""
    v = vec
    for name, (_, scale, causal) in CASES.items():
        y = cf.softmax_bias_fwd(v[name + "_x"], v[name + "_m"], scale, causal=causal)
        assert np.allclose(y, v[name + "_y"], rtol=2e-6, atol=1e-12), name
        exact = cf.softmax_bias_fwd(v[name + "_x"], v[name + "_m"], scale, causal=causal, sum_f32=False)
        assert np.allclose(exact, v[name + "_y"], rtol=1e-12, atol=1e-300), name
        dx = cf.softmax_bwd(v[name + "_g"], v[name + "_y"], scale)
        assert np.allclose(dx, v[name + "_dx"], rtol=1e-10, atol=1e-14), name
    # the gradient of a broadcast term is the gradient of the sum, reduced
    assert np.allclose(v["t5_dm"], (v["t5_dx"] / 1.0).sum(0, keepdims=True), rtol=1e-12, atol=1e-14)
    keep = philox.keep_mask(v["drop_x"].size, DROP["p"], DROP["seed"], DROP["offset"]).reshape(v["drop_x"].shape)
    assert np.array_equal(keep, v["drop_keep"])
    out = cf.softmax_bias_dropout_fwd(v["drop_x"], v["drop_m"], DROP["scale"], keep, DROP["p"])
    assert np.allclose(out, v["drop_out"], rtol=2e-6, atol=1e-12)
    dx = cf.softmax_bias_dropout_bwd(v["drop_g"], v["drop_x"], v["drop_m"], DROP["scale"], keep, DROP["p"])
    assert np.allclose(dx, v["drop_dx"], rtol=2e-6, atol=1e-10)


def test_vectors_satisfy_the_invariants(vec):
    v = vec
    for name in CASES:
        assert np.allclose(v[name + "_y"].sum(-1), 1.0, atol=1e-12)
        assert np.allclose(v[name + "_dx"].sum(-1), 0.0, atol=1e-12)
    # keys behind the diagonal and behind a fill are exact zeros in float64 already
    assert np.all(np.triu(v["gpt2_y"], 1 + 64 - 16) == 0) and np.all(v["gpt2_y"][1, ..., 40:] == 0)
    assert np.all(v["bart_y"][np.broadcast_to(v["bart_m"] < 0, v["bart_y"].shape)] == 0)
    assert np.all(v["drop_out"][v["drop_keep"] == 0] == 0)


def T(a, dtype, device):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).to(device)


@pytest.mark.gpu
def test_kernels_match_the_committed_vectors(device, vec):
    from oslo_amd.torch import _C

    v = vec
    k = _C.get_softmax_kernel()
    for name, (dtype, scale, causal) in CASES.items():
        x, m, g = (T(v[name + "_" + t], dtype, device) for t in "xmg")
        for skip in (False, True):
            y = k.softmax_bias_forward(x, m, scale, causal=causal, skip_hidden=skip)
            check(y, v[name + "_y"], name + " fwd", atol=1e-9)
            dx = k.softmax_bias_backward(g, y, scale, bias=m, causal=causal, skip_hidden=skip)
            # (the kernel differentiates through the stored, rounded probabilities)
            check(dx, cf.softmax_bwd(v[name + "_g"], np.asarray(y.double().cpu()), scale), name + " bwd", atol=1e-7)
            if dtype == torch.float32:
                check(dx, v[name + "_dx"], name + " bwd against torch", atol=2e-7)
    # the learned term's gradient through the autograd Function
    import oslo_amd.torch.nn as onn
    x = T(v["t5_x"], torch.float32, device).requires_grad_()
    m = T(v["t5_m"], torch.float32, device).requires_grad_()
    onn.scaled_bias_softmax(x, m, 1.0).backward(T(v["t5_g"], torch.float32, device))
    check(m.grad, v["t5_dm"], "t5 dM", atol=1e-6)
    check(x.grad, v["t5_dx"], "t5 dx", atol=2e-7)
    # fused dropout
    x, m, g = (T(v["drop_" + t], DROP["dtype"], device) for t in "xmg")
    out, stats = k.softmax_bias_dropout_forward(x, m, DROP["scale"], DROP["p"], DROP["seed"], DROP["offset"])
    check(out, v["drop_out"], "dropout fwd", atol=1e-9)
    assert (out.cpu()[torch.from_numpy(v["drop_keep"] == 0)] == 0).all()
    dx = k.softmax_bias_dropout_backward(g, x, m, stats, DROP["scale"], DROP["p"], DROP["seed"], DROP["offset"])
    check(dx, v["drop_dx"], "dropout bwd", atol=2e-7)
