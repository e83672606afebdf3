"""Writes tests/golden/hot_path_vectors.npz: small seeded inputs and the outputs
of the float64 oracle (oracle/closed_form.py, oracle/philox.py) for every op.

    python tests/golden/make_fixtures.py

The reference repository holds no numeric fixture for this path (its tests draw
unseeded random data), so these vectors pin the oracle and the kernels against
regressions; what pins the oracle itself is tests/test_oracle_*.py.  Inputs are
stored as the exact values of the storage type (float32 arrays holding bf16 /
fp16-representable numbers), expected outputs as float64.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import closed_form as cf  # noqa: E402
from oracle import philox  # noqa: E402


def main():
    r = np.random.default_rng(20240611)
    out = {}

    def bf16(a):
        return cf.round_bf16(a.astype(np.float32))

    def f16(a):
        return cf.round_f16(a.astype(np.float32))

    # LayerNorm / RMSNorm, bf16, [8, 256]
    x = bf16(r.standard_normal((8, 256)) * 1.3 + 0.2)
    gamma = bf16(1 + 0.02 * r.standard_normal(256))
    beta = bf16(0.02 * r.standard_normal(256))
    dy = bf16(r.standard_normal((8, 256)))
    y, mean, invvar = cf.layer_norm_fwd(x, gamma, beta, 1e-5)
    dx, dg, db = cf.layer_norm_bwd(dy, x, mean, invvar, gamma)
    out.update(ln_x=x, ln_gamma=gamma, ln_beta=beta, ln_dy=dy, ln_y=y, ln_mean=mean, ln_invvar=invvar,
               ln_dx=dx, ln_dgamma=dg, ln_dbeta=db)
    ry, rinv = cf.rms_norm_fwd(x, gamma, 1e-5, out="bf16")
    rdx, rdg = cf.rms_norm_bwd(dy, x, rinv, gamma)
    out.update(rms_y=np.asarray(ry, dtype=np.float64), rms_invvar=rinv, rms_dx=rdx, rms_dgamma=rdg)

    # causal softmax, fp32, [2, 16, 16], scale 0.125
    sx = r.standard_normal((2, 16, 16)).astype(np.float32)
    sg = r.standard_normal((2, 16, 16)).astype(np.float32)
    sy = cf.softmax_causal_fwd(sx, 0.125)
    out.update(sm_x=sx, sm_g=sg, sm_y=sy, sm_dx=cf.softmax_bwd(sg, sy, 0.125))

    # padding-masked softmax, fp16, [2, 2, 4, 64], valid lengths 64 and 23
    mx = f16(2 * r.standard_normal((2, 2, 4, 64)))
    mg = f16(r.standard_normal((2, 2, 4, 64)))
    pad = np.arange(64)[None, :] >= np.array([64, 23])[:, None]
    my = cf.softmax_masked_fwd(mx, pad[:, None, None, :], 0.125)
    out.update(msm_x=mx, msm_g=mg, msm_pad=pad, msm_y=my, msm_dx=cf.softmax_bwd(mg, my, 0.125))

    # bias-GeLU, bf16, [4, 64]
    gx = bf16(r.standard_normal((4, 64)) * 1.5)
    gb = bf16(0.3 * r.standard_normal(64))
    gg = bf16(r.standard_normal((4, 64)))
    gdx, gdb = cf.bias_gelu_bwd(gg, gx, gb, out="bf16")
    out.update(gelu_x=gx, gelu_b=gb, gelu_g=gg, gelu_y=cf.bias_gelu_fwd(gx, gb),
               gelu_dx=np.asarray(gdx, dtype=np.float64), gelu_db=np.asarray(gdb, dtype=np.float64))

    # bias-dropout-add, bf16, [4, 64], p = 0.1, Philox seed 1234, offset 8
    bx = bf16(r.standard_normal((4, 64)))
    bb = bf16(0.02 * r.standard_normal(64))
    br = bf16(r.standard_normal((4, 64)))
    bg = bf16(r.standard_normal((4, 64)))
    keep = philox.keep_mask(256, 0.1, 1234, 8).reshape(4, 64)
    bdx, bdb = cf.bias_dropout_add_bwd(bg, keep, 0.1, out="bf16")
    out.update(bda_x=bx, bda_b=bb, bda_res=br, bda_g=bg, bda_keep=keep,
               bda_out=cf.bias_dropout_add_fwd(bx, bb, br, keep, 0.1),
               bda_dx=np.asarray(bdx, dtype=np.float64), bda_db=np.asarray(bdb, dtype=np.float64))

    # raw Philox words: groups 0..3 and 2^32-2..2^32+1 for (seed, offset) = (1234, 8)
    out.update(philox_lo=philox.group_words(0, 4, 1234, 8), philox_hi=philox.group_words(2 ** 32 - 2, 4, 1234, 8))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_path_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
