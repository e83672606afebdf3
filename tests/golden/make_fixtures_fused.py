"""Writes tests/golden/fused_ops_vectors.npz: small seeded inputs and the float64
oracle's outputs for the ops added around the hot path -- softmax with fused
dropout, bias-dropout-add fused into LayerNorm, the Adam / AdamW step.

    python tests/golden/make_fixtures_fused.py

Same conventions as make_fixtures.py: inputs hold the exact values of their
storage type, expected outputs are float64 (rounded to the storage type where
the kernel stores an intermediate).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import closed_form as cf  # noqa: E402
from oracle import philox  # noqa: E402


def main():
    r = np.random.default_rng(20240923)
    out = {}

    def bf16(a):
        return cf.round_bf16(a.astype(np.float32))

    # causal softmax + dropout, bf16, [2, 16, 32], scale 0.25, p 0.2, Philox (77, 12)
    x = bf16(r.standard_normal((2, 16, 32)))
    g = bf16(r.standard_normal((2, 16, 32)))
    keep = philox.keep_mask(x.size, 0.2, 77, 12).reshape(x.shape)
    hidden = cf.causal_hidden(16, 32)
    out.update(smd_x=x, smd_g=g, smd_keep=keep,
               smd_out=cf.softmax_dropout_fwd(x, hidden, 0.25, keep, 0.2),
               smd_dx=cf.softmax_dropout_bwd(g, x, hidden, 0.25, keep, 0.2))

    # bias-dropout-add + LayerNorm, bf16, [6, 128], p 0.1, Philox (1234, 8)
    fx = bf16(r.standard_normal((6, 128)))
    fb = bf16(0.1 * r.standard_normal(128))
    fr = bf16(r.standard_normal((6, 128)))
    fg = bf16(1 + 0.1 * r.standard_normal(128))
    fbeta = bf16(0.1 * r.standard_normal(128))
    fdy = bf16(r.standard_normal((6, 128)))
    fdh = bf16(r.standard_normal((6, 128)))
    fkeep = philox.keep_mask(fx.size, 0.1, 1234, 8).reshape(fx.shape)
    y, h, mean, invvar = cf.bias_dropout_add_norm_fwd(fx, fb, fr, fkeep, 0.1, fg, fbeta, 1e-5, False, "bf16")
    dres, dx, dgam, dbet, dbias = cf.bias_dropout_add_norm_bwd(fdy, fdh, h, mean, invvar, fg, fkeep, 0.1, False, "bf16")
    out.update(fln_x=fx, fln_bias=fb, fln_res=fr, fln_gamma=fg, fln_beta=fbeta, fln_dy=fdy, fln_dh=fdh,
               fln_keep=fkeep, fln_y=np.asarray(y, np.float64), fln_h=np.asarray(h, np.float64),
               fln_mean=mean, fln_invvar=invvar, fln_dres=np.asarray(dres, np.float64),
               fln_dx=np.asarray(dx, np.float64), fln_dgamma=np.asarray(dgam, np.float64),
               fln_dbeta=np.asarray(dbet, np.float64), fln_dbias=np.asarray(dbias, np.float64))

    # AdamW and Adam (L2), fp32, 300 elements, step 3
    ag = r.standard_normal(300).astype(np.float32)
    ap = r.standard_normal(300).astype(np.float32)
    am = (0.1 * r.standard_normal(300)).astype(np.float32)
    av = np.abs(0.1 * r.standard_normal(300)).astype(np.float32)
    for mode, tag in ((1, "adamw"), (0, "adaml2")):
        p, m, v = cf.adam_step(ag, ap, am, av, 1e-2, 0.9, 0.999, 1e-8, 3, mode, True, 0.05)
        out.update({tag + "_p": p, tag + "_m": m, tag + "_v": v})
    out.update(adam_g=ag, adam_p=ap, adam_m=am, adam_v=av)

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fused_ops_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
