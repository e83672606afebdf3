"""Writes tests/golden/optimizer_vectors.npz: small seeded inputs and the float64
oracle's outputs for the multi-tensor optimizer steps besides Adam -- SGD,
Adagrad, NovoGrad, LAMB (both stages) and the tensor norms.

    python tests/golden/make_fixtures_optimizers.py

fp32 inputs, 300 elements per tensor; the hyper-parameters are stored with the
vectors so that a reader needs nothing but the file.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import closed_form as cf  # noqa: E402

HYPER = dict(lr=0.0625, wd=0.03125, momentum=0.875, dampening=0.25, eps=2.0 ** -20, beta1=0.875, beta2=0.96875,
             step=3, scale=0.5, max_grad_norm=4.0)


def main():
    r = np.random.default_rng(20250101)
    h = HYPER
    f32 = lambda a: a.astype(np.float32)
    g, p = f32(r.standard_normal(300)), f32(r.standard_normal(300))
    m, v = f32(0.1 * r.standard_normal(300)), f32(np.abs(0.1 * r.standard_normal(300)))
    out = dict(g=g, p=p, m=m, v=v, **{"hyper_" + k: np.float64(x) for k, x in h.items()})

    # SGD: momentum with dampening, decay after the momentum step, a gradient scale
    w, mom, _ = cf.sgd_step(g, p, m, h["lr"], h["wd"], h["momentum"], h["dampening"], False, False,
                            wd_after_momentum=True, scale=h["scale"])
    out.update(sgd_w=w, sgd_mom=mom)
    w, mom, _ = cf.sgd_step(g, p, m, h["lr"], h["wd"], h["momentum"], 0.0, True, True)
    out.update(sgd_first_nesterov_w=w, sgd_first_nesterov_mom=mom)

    # Adagrad: L2 and decoupled decay
    for mode in (0, 1):
        pp, hh = cf.adagrad_step(g, p, v, h["lr"], h["eps"], mode, h["wd"])
        out.update({"adagrad%d_p" % mode: pp, "adagrad%d_h" % mode: hh})

    # norms and their blends
    out.update(norm_l2=np.float64(cf.tensor_norm(g, 2)), norm_max=np.float64(cf.tensor_norm(g, 0)),
               blend_l2=np.float64(cf.blend_norm(1.5, g, h["beta2"], 1.0 - h["beta2"], 2)),
               blend_max=np.float64(cf.blend_norm(1.5, g, h["beta2"], 1.0 - h["beta2"], 0)))

    # NovoGrad: both moment modes, from the blended L2 norm above
    for mode in (0, 1):
        pp, mm = cf.novograd_step(g, p, m, np.float32(out["blend_l2"]), h["lr"], h["beta1"], h["beta2"], h["eps"],
                                  h["step"], True, h["wd"], True, mode)
        out.update({"novograd%d_p" % mode: pp, "novograd%d_m" % mode: mm})

    # LAMB: the gradient norm (17.x) exceeds the threshold 4, so the gradient is clipped
    gn = np.float32(cf.tensor_norm(g, 2))
    for mode in (0, 1):
        u, mm, vv = cf.lamb_stage1(g, p, m, v, h["beta1"], h["beta2"], h["eps"], h["step"], True, h["wd"], True,
                                   mode, gn, h["max_grad_norm"])
        pp = cf.lamb_stage2(u, p, np.float32(cf.tensor_norm(p)), np.float32(cf.tensor_norm(u)), h["lr"], h["wd"],
                            False)
        out.update({"lamb%d_update" % mode: u, "lamb%d_m" % mode: mm, "lamb%d_v" % mode: vv,
                    "lamb%d_p" % mode: pp})

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "optimizer_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
