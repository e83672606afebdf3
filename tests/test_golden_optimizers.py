"""Committed vectors of the optimizer steps (tests/golden/optimizer_vectors.npz,
written by tests/golden/make_fixtures_optimizers.py): the oracle still
reproduces them (no GPU), and the kernels match them through the C ABI."""
import os

import numpy as np
import pytest
import torch

from helpers import check
from oracle import closed_form as cf

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "optimizer_vectors.npz")


@pytest.fixture(scope="module")
def vec():
    with np.load(PATH) as z:
        return {k: z[k] for k in z.files}


def hyper(v):
    return {k[6:]: float(v[k]) for k in v if k.startswith("hyper_")}


def test_oracle_reproduces_the_committed_vectors(vec):
    v, h = vec, hyper(vec)
    w, mom, _ = cf.sgd_step(v["g"], v["p"], v["m"], h["lr"], h["wd"], h["momentum"], h["dampening"], False, False,
                            wd_after_momentum=True, scale=h["scale"])
    assert np.array_equal(w, v["sgd_w"]) and np.array_equal(mom, v["sgd_mom"])
    for mode in (0, 1):
        p, hh = cf.adagrad_step(v["g"], v["p"], v["v"], h["lr"], h["eps"], mode, h["wd"])
        assert np.array_equal(p, v["adagrad%d_p" % mode]) and np.array_equal(hh, v["adagrad%d_h" % mode])
        p, m = cf.novograd_step(v["g"], v["p"], v["m"], np.float32(v["blend_l2"]), h["lr"], h["beta1"], h["beta2"],
                                h["eps"], int(h["step"]), True, h["wd"], True, mode)
        assert np.array_equal(p, v["novograd%d_p" % mode]) and np.array_equal(m, v["novograd%d_m" % mode])
        u, m, s = cf.lamb_stage1(v["g"], v["p"], v["m"], v["v"], h["beta1"], h["beta2"], h["eps"], int(h["step"]),
                                 True, h["wd"], True, mode, np.float32(cf.tensor_norm(v["g"])), h["max_grad_norm"])
        assert np.array_equal(u, v["lamb%d_update" % mode])
    assert float(cf.tensor_norm(v["g"], 2)) == float(v["norm_l2"])
    assert float(cf.tensor_norm(v["g"])) > h["max_grad_norm"]  # the LAMB vectors are clipped ones


@pytest.mark.gpu
def test_kernels_match_the_committed_vectors(device, vec):
    from oslo_amd.torch import _C

    v, h = vec, hyper(vec)
    T = lambda name: torch.from_numpy(np.ascontiguousarray(v[name], dtype=np.float32)).to(device)
    step = int(h["step"])

    lists = [[T("g")], [T("p")], [T("m")]]
    _C.get_sgd_kernel().multi_tensor_sgd(0, None, lists, h["wd"], h["momentum"], h["dampening"], h["lr"], False,
                                         False, True, h["scale"])
    check(lists[1][0], v["sgd_w"], "golden sgd w")
    check(lists[2][0], v["sgd_mom"], "golden sgd momentum")
    lists = [[T("g")], [T("p")], [T("m")]]
    _C.get_sgd_kernel().multi_tensor_sgd(0, None, lists, h["wd"], h["momentum"], 0.0, h["lr"], True, True, False, 1.0)
    check(lists[1][0], v["sgd_first_nesterov_w"], "golden sgd (first run, Nesterov) w")
    check(lists[2][0], v["sgd_first_nesterov_mom"], "golden sgd (first run, Nesterov) momentum")

    for mode in (0, 1):
        lists = [[T("g")], [T("p")], [T("v")]]
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, None, lists, h["lr"], h["eps"], mode, h["wd"])
        check(lists[1][0], v["adagrad%d_p" % mode], "golden adagrad p (mode %d)" % mode)
        check(lists[2][0], v["adagrad%d_h" % mode], "golden adagrad h (mode %d)" % mode, atol=1e-8)

    norms = _C.get_l2norm_kernel()
    total, per = norms.multi_tensor_l2norm(0, None, [[T("g")]], True)
    assert np.isclose(total.item(), float(v["norm_l2"]), rtol=2e-6) and np.isclose(per.item(), float(v["norm_l2"]), rtol=2e-6)
    for norm_type, key in ((2, "blend_l2"), (0, "blend_max")):
        out = torch.full((1,), 1.5, device=device)
        norms.multi_tensor_norm_out(0, None, [[T("g")]], out, h["beta2"], 1.0 - h["beta2"], norm_type)
        assert np.isclose(out.item(), float(v[key]), rtol=2e-6), key

    for mode in (0, 1):
        lists = [[T("g")], [T("p")], [T("m")]]
        stored = torch.full((1,), 1.5, device=device)
        _C.get_novograd_kernel().multi_tensor_novograd(0, None, lists, stored, h["lr"], h["beta1"], h["beta2"],
                                                       h["eps"], step, 1, h["wd"], 1, mode, 2)
        check(lists[1][0], v["novograd%d_p" % mode], "golden novograd p (mode %d)" % mode, atol=2e-6)
        check(lists[2][0], v["novograd%d_m" % mode], "golden novograd m (mode %d)" % mode)

        lists = [[T("g")], [T("p")], [T("m")], [T("v")]]
        gnorm, _ = norms.multi_tensor_l2norm(0, None, [lists[0]], False)
        _C.get_lamb_kernel().multi_tensor_lamb(0, None, lists, h["lr"], h["beta1"], h["beta2"], h["eps"], step, 1,
                                               h["wd"], 1, mode, gnorm, h["max_grad_norm"], False)
        check(lists[0][0], v["lamb%d_update" % mode], "golden lamb update (mode %d)" % mode)
        check(lists[2][0], v["lamb%d_m" % mode], "golden lamb m (mode %d)" % mode, atol=1e-7)
        check(lists[3][0], v["lamb%d_v" % mode], "golden lamb v (mode %d)" % mode, atol=1e-8)
        check(lists[1][0], v["lamb%d_p" % mode], "golden lamb p (mode %d)" % mode, atol=2e-6)
