"""Committed vectors (tests/golden/hot_path_vectors.npz, written by
tests/golden/make_fixtures.py): the oracle must keep reproducing them (CPU), and
the HIP kernels must match them through the C ABI (GPU)."""
import os

import numpy as np
import pytest
import torch

from helpers import check, check_f32
from oracle import closed_form as cf
from oracle import philox

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hot_path_vectors.npz")


@pytest.fixture(scope="module")
def vec():
    return dict(np.load(PATH, allow_pickle=False))


def test_oracle_reproduces_committed_vectors(vec):
    v = vec
    y, mean, invvar = cf.layer_norm_fwd(v["ln_x"], v["ln_gamma"], v["ln_beta"], 1e-5)
    assert np.array_equal(y, v["ln_y"]) and np.array_equal(mean, v["ln_mean"])
    dx, dg, db = cf.layer_norm_bwd(v["ln_dy"], v["ln_x"], mean, invvar, v["ln_gamma"])
    assert np.array_equal(dx, v["ln_dx"]) and np.array_equal(dg, v["ln_dgamma"]) and np.array_equal(db, v["ln_dbeta"])
    ry, rinv = cf.rms_norm_fwd(v["ln_x"], v["ln_gamma"], 1e-5, out="bf16")
    assert np.array_equal(np.asarray(ry, dtype=np.float64), v["rms_y"])
    sy = cf.softmax_causal_fwd(v["sm_x"], 0.125)
    assert np.array_equal(sy, v["sm_y"])
    assert np.array_equal(cf.softmax_bwd(v["sm_g"], sy, 0.125), v["sm_dx"])
    my = cf.softmax_masked_fwd(v["msm_x"], v["msm_pad"][:, None, None, :], 0.125)
    assert np.array_equal(my, v["msm_y"])
    assert np.array_equal(cf.bias_gelu_fwd(v["gelu_x"], v["gelu_b"]), v["gelu_y"])
    keep = philox.keep_mask(256, 0.1, 1234, 8).reshape(4, 64)
    assert np.array_equal(keep, v["bda_keep"])
    assert np.array_equal(cf.bias_dropout_add_fwd(v["bda_x"], v["bda_b"], v["bda_res"], keep, 0.1), v["bda_out"])
    assert np.array_equal(philox.group_words(0, 4, 1234, 8), v["philox_lo"])
    assert np.array_equal(philox.group_words(2 ** 32 - 2, 4, 1234, 8), v["philox_hi"])


def test_vectors_satisfy_the_invariants(vec):
    v = vec
    assert np.allclose(v["sm_y"].sum(-1), 1) and np.all(np.triu(v["sm_y"], 1) == 0)
    assert np.all(v["msm_y"][1][..., 23:] == 0) and np.allclose(v["msm_y"].sum(-1), 1)
    assert np.allclose(v["ln_dbeta"], v["ln_dy"].sum(0))
    assert np.allclose(v["ln_dx"].sum(-1), 0, atol=1e-12)
    assert np.array_equal(v["bda_out"][v["bda_keep"] == 0], v["bda_res"][v["bda_keep"] == 0].astype(np.float64))


def T(a, dtype, device):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).to(device)


@pytest.mark.gpu
def test_kernels_match_committed_vectors(device, vec):
    from oslo_amd.torch import _C

    v = vec
    BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32
    ln = _C.get_layernorm_kernel()
    x, g, b, dy = (T(v[k], BF16, device) for k in ("ln_x", "ln_gamma", "ln_beta", "ln_dy"))
    y, mean, invvar = ln.layer_norm_forward_affine(x, (256,), g, b, 1e-5)
    check(y, v["ln_y"], "golden ln fwd")
    check_f32(mean, v["ln_mean"], "golden ln mean", atol=2e-6)
    check_f32(invvar, v["ln_invvar"], "golden ln invvar", atol=0)
    dx, dg, db = ln.layer_norm_backward_affine(dy, mean, invvar, x, (256,), g, b, 1e-5)
    check(dx, v["ln_dx"], "golden ln dx", atol=4e-6)
    check(dg, v["ln_dgamma"], "golden ln dgamma", atol=3e-5, min_exact=0.97)
    check(db, v["ln_dbeta"], "golden ln dbeta", atol=3e-5, min_exact=0.97)
    y, invvar = ln.rms_norm_forward_affine(x, (256,), g, 1e-5)
    check(y, v["rms_y"], "golden rms fwd", max_ulp=2, min_exact=0.995)
    dx, dg = ln.rms_norm_backward_affine(dy, invvar, x, (256,), g, 1e-5)
    check(dx, v["rms_dx"], "golden rms dx", atol=4e-6)
    check(dg, v["rms_dgamma"], "golden rms dgamma", atol=3e-5, min_exact=0.97)

    sm = _C.get_softmax_kernel()
    y = sm.fused_scaled_upper_triang_masked_softmax_forward(T(v["sm_x"], F32, device), 0.125)
    check(y, v["sm_y"], "golden causal fwd", atol=1e-9)
    dx = sm.fused_scaled_upper_triang_masked_softmax_backward(T(v["sm_g"], F32, device), T(v["sm_y"], F32, device), 0.125)
    check(dx, v["sm_dx"], "golden causal bwd", atol=1e-7)
    mask = torch.from_numpy(v["msm_pad"]).view(2, 1, 1, 64).to(device)
    y = sm.fused_scaled_masked_softmax_forward(T(v["msm_x"], F16, device), mask, 0.125)
    check(y, v["msm_y"], "golden masked fwd", atol=1e-9)

    el = _C.get_fused_elementwise_kernel()
    gx, gb, gg = (T(v[k], BF16, device) for k in ("gelu_x", "gelu_b", "gelu_g"))
    check(el.bias_gelu_forward(gx, gb), v["gelu_y"], "golden gelu fwd")
    dx, db = el.bias_gelu_backward(gg, gx, gb)
    check(dx, v["gelu_dx"], "golden gelu dx")
    check(db, v["gelu_db"], "golden gelu dbias", atol=1e-4, min_exact=0.9)
    bx, bb, br, bg = (T(v[k], BF16, device) for k in ("bda_x", "bda_b", "bda_res", "bda_g"))
    out, mask = el.bias_dropout_add_forward(bx, bb, br, 0.1, 1234, 8, return_mask=True)
    assert np.array_equal(mask.cpu().numpy(), v["bda_keep"])
    check(out, v["bda_out"], "golden bda fwd", atol=1e-6)
    dx, db = el.bias_dropout_add_backward(bg, 0.1, 1234, 8)
    check(dx, v["bda_dx"], "golden bda dx")
    check(db, v["bda_db"], "golden bda dbias", atol=1e-4, min_exact=0.9)
    words = el.philox_words(4, 0, 1234, 8, device).cpu().numpy().view(np.uint32).reshape(4, 4)
    assert np.array_equal(words, v["philox_lo"])
    words = el.philox_words(4, 2 ** 32 - 2, 1234, 8, device).cpu().numpy().view(np.uint32).reshape(4, 4)
    assert np.array_equal(words, v["philox_hi"])
