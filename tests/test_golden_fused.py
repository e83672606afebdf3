"""Committed vectors of the fused ops (tests/golden/fused_ops_vectors.npz, written
by tests/golden/make_fixtures_fused.py): the oracle must keep reproducing them
(CPU) and the HIP kernels must match them through the C ABI (GPU)."""
import os

import numpy as np
import pytest
import torch

from helpers import check
from oracle import closed_form as cf
from oracle import philox

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fused_ops_vectors.npz")


@pytest.fixture(scope="module")
def vec():
    return dict(np.load(PATH, allow_pickle=False))


def test_oracle_reproduces_committed_vectors(vec):
    v = vec
    keep = philox.keep_mask(v["smd_x"].size, 0.2, 77, 12).reshape(v["smd_x"].shape)
    assert np.array_equal(keep, v["smd_keep"])
    hidden = cf.causal_hidden(16, 32)
    assert np.array_equal(cf.softmax_dropout_fwd(v["smd_x"], hidden, 0.25, keep, 0.2), v["smd_out"])
    assert np.array_equal(cf.softmax_dropout_bwd(v["smd_g"], v["smd_x"], hidden, 0.25, keep, 0.2), v["smd_dx"])
    fkeep = philox.keep_mask(v["fln_x"].size, 0.1, 1234, 8).reshape(v["fln_x"].shape)
    assert np.array_equal(fkeep, v["fln_keep"])
    y, h, mean, invvar = cf.bias_dropout_add_norm_fwd(
        v["fln_x"], v["fln_bias"], v["fln_res"], fkeep, 0.1, v["fln_gamma"], v["fln_beta"], 1e-5, False, "bf16")
    assert np.array_equal(np.asarray(y, np.float64), v["fln_y"]) and np.array_equal(np.asarray(h, np.float64), v["fln_h"])
    dres, dx, dg, db, dbias = cf.bias_dropout_add_norm_bwd(
        v["fln_dy"], v["fln_dh"], h, mean, invvar, v["fln_gamma"], fkeep, 0.1, False, "bf16")
    for got, key in ((dres, "fln_dres"), (dx, "fln_dx"), (dg, "fln_dgamma"), (db, "fln_dbeta"), (dbias, "fln_dbias")):
        assert np.array_equal(np.asarray(got, np.float64), v[key]), key
    for mode, tag in ((1, "adamw"), (0, "adaml2")):
        p, m, vv = cf.adam_step(v["adam_g"], v["adam_p"], v["adam_m"], v["adam_v"], 1e-2, 0.9, 0.999, 1e-8, 3,
                                mode, True, 0.05)
        assert np.array_equal(p, v[tag + "_p"]) and np.array_equal(m, v[tag + "_m"]) and np.array_equal(vv, v[tag + "_v"])


def test_vectors_satisfy_the_invariants(vec):
    v = vec
    drop = v["smd_keep"] == 0
    assert np.all(v["smd_out"][drop] == 0) and np.all(np.triu(v["smd_out"], 1 + 32 - 16) == 0)
    # kept probabilities, unscaled, sum to at most 1 per row and the gradient rows sum to 0
    assert np.all((v["smd_out"] * 0.8).sum(-1) <= 1 + 1e-6)
    assert np.allclose(v["smd_dx"].sum(-1), 0, atol=1e-12)
    fdrop = v["fln_keep"] == 0
    assert np.array_equal(v["fln_h"][fdrop], v["fln_res"][fdrop].astype(np.float64))
    assert np.all(v["fln_dx"][fdrop] == 0)
    assert np.allclose(v["fln_dbias"], v["fln_dx"].sum(0), rtol=2 ** -7)
    # AdamW and Adam-L2 share nothing but the inputs once the decay is non-zero
    assert not np.allclose(v["adamw_m"], v["adaml2_m"]) and not np.allclose(v["adamw_p"], v["adaml2_p"])


def T(a, dtype, device):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).to(device)


@pytest.mark.gpu
def test_kernels_match_committed_vectors(device, vec):
    from oslo_amd.torch import _C

    v = vec
    BF16, F32 = torch.bfloat16, torch.float32
    sm = _C.get_softmax_kernel()
    x, g = T(v["smd_x"], BF16, device), T(v["smd_g"], BF16, device)
    out, stats = sm.softmax_dropout_forward(x, None, 0.25, 0.2, 77, 12)
    check(out, v["smd_out"], "golden softmax-dropout fwd", atol=1e-9)
    assert torch.equal(out.cpu() != 0, torch.from_numpy((v["smd_keep"] != 0) & (v["smd_out"] != 0)))
    dx = sm.softmax_dropout_backward(g, x, stats, None, 0.25, 0.2, 77, 12)
    check(dx, v["smd_dx"], "golden softmax-dropout bwd", atol=2e-7)

    ln = _C.get_layernorm_kernel()
    t = {k: T(v["fln_" + k], BF16, device) for k in ("x", "bias", "res", "gamma", "beta", "dy", "dh")}
    y, h, mean, invvar = ln.bias_dropout_add_norm_forward(
        False, t["x"], t["bias"], t["res"], (128,), t["gamma"], t["beta"], 1e-5, 0.1, 1234, 8)
    check(h, v["fln_h"], "golden fused h", atol=1e-6)
    check(y, v["fln_y"], "golden fused y", atol=1e-2, min_exact=0.97)
    hk = T(v["fln_h"], BF16, device)
    dres, dxx, dg, db, dbias = ln.bias_dropout_add_norm_backward(
        False, t["dy"], t["dh"], hk, T(v["fln_mean"], F32, device), T(v["fln_invvar"], F32, device),
        (128,), t["gamma"], 0.1, 1234, 8)
    check(dres, v["fln_dres"], "golden fused dres", atol=2e-6)
    check(dxx, v["fln_dx"], "golden fused dx", atol=2e-6)
    check(dg, v["fln_dgamma"], "golden fused dgamma", atol=3e-5, min_exact=0.97, max_ulp=2)
    check(db, v["fln_dbeta"], "golden fused dbeta", atol=3e-5, min_exact=0.97, max_ulp=2)
    check(dbias, v["fln_dbias"], "golden fused dbias", atol=3e-5, min_exact=0.97, max_ulp=2)

    ad = _C.get_adam_kernel()
    for mode, tag in ((1, "adamw"), (0, "adaml2")):
        lists = [[T(v["adam_" + k], F32, device)] for k in ("g", "p", "m", "v")]
        ad.multi_tensor_adam(0, None, lists, 1e-2, 0.9, 0.999, 1e-8, 3, mode, 1, 0.05)
        check(lists[1][0], v[tag + "_p"], "golden %s p" % tag, atol=5e-7)
        check(lists[2][0], v[tag + "_m"], "golden %s m" % tag, atol=1e-7)
        check(lists[3][0], v[tag + "_v"], "golden %s v" % tag, atol=1e-8)
