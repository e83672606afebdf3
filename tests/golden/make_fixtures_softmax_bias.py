"""Writes tests/golden/softmax_bias_vectors.npz: small seeded inputs of the softmax
with an additive floating-point term, y = softmax(scale * x + M), and what torch
returns for the unfused chain on them in float64 on the CPU (forward, and the
gradients of the scores and of the term by autograd).  The expected values come
from torch, not from oracle/: the oracle and the kernels are both checked against
them.

    python tests/golden/make_fixtures_softmax_bias.py

The chains are the reference's call sites: the -10000 key mask of
oslo/transformers/models/bert/modeling_bert.py:298-306 (here with GPT-2's causal
`where` on top, models/gpt2/modeling_gpt2.py:126-136), the finfo.min mask of
models/bart/modeling_bart.py:123-136, the position bias of
models/t5/modeling_t5.py:508-514, and softmax followed by dropout
(modeling_bert.py:306-310) with the keep decisions of the library's Philox stream.
Inputs hold exact values of their storage type.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import philox  # noqa: E402  (the keep bits only: pinned by the Random123 vectors)


def rounded(a, dtype):
    return torch.from_numpy(a.astype(np.float32)).to(dtype).double()


def chain(x, m, g, scale, causal_fill=None, keep=None, p=0.0):
    x = x.clone().requires_grad_()
    m = m.clone().requires_grad_()
    s = scale * x + m
    if causal_fill is not None:
        sq, sk = x.shape[-2:]
        hidden = torch.ones(sq, sk, dtype=torch.bool).triu(1 + sk - sq)
        s = s.masked_fill(hidden, causal_fill)
    y = torch.softmax(s, dim=-1)
    out = y if keep is None else y * keep / (1.0 - p)
    out.backward(g)
    return out.detach().numpy(), x.grad.numpy(), m.grad.numpy()


def main():
    r = np.random.default_rng(20250117)
    out = {}

    # GPT-2: causal + additive -10000 key mask [b,1,1,sk], bf16, [2,2,16,64], scale 0.125
    x = rounded(2 * r.standard_normal((2, 2, 16, 64)), torch.bfloat16)
    g = rounded(r.standard_normal((2, 2, 16, 64)), torch.bfloat16)
    m = torch.zeros(2, 1, 1, 64, dtype=torch.float64)
    m[1, ..., 40:] = -10000.0
    y, dx, _ = chain(x, m, g, 0.125, causal_fill=float("-inf"))
    out.update(gpt2_x=x.numpy(), gpt2_m=m.numpy(), gpt2_g=g.numpy(), gpt2_y=y, gpt2_dx=dx)

    # BART: finfo.min mask per query [b,1,sq,sk], fp16, [2,3,8,128], scale 0.25
    x = rounded(2 * r.standard_normal((2, 3, 8, 128)), torch.float16)
    g = rounded(r.standard_normal((2, 3, 8, 128)), torch.float16)
    cut = torch.from_numpy(r.integers(1, 129, size=(2, 1, 8, 1)))
    m = torch.zeros(2, 1, 8, 128, dtype=torch.float64).masked_fill(
        torch.arange(128).view(1, 1, 1, 128) >= cut, float(torch.finfo(torch.float16).min))
    y, dx, _ = chain(x, m, g, 0.25)
    out.update(bart_x=x.numpy(), bart_m=m.numpy(), bart_g=g.numpy(), bart_y=y, bart_dx=dx)

    # T5: learned position bias [1,np,sq,sk], fp32, [3,2,24,24], scale 1
    x = rounded(2 * r.standard_normal((3, 2, 24, 24)), torch.float32)
    g = rounded(r.standard_normal((3, 2, 24, 24)), torch.float32)
    m = rounded(1.5 * r.standard_normal((1, 2, 24, 24)), torch.float32)
    y, dx, dm = chain(x, m, g, 1.0)
    out.update(t5_x=x.numpy(), t5_m=m.numpy(), t5_g=g.numpy(), t5_y=y, t5_dx=dx, t5_dm=dm)

    # BERT with attention dropout: -10000 key mask, bf16, [2,2,8,96], scale 0.125, p 0.2, Philox (31, 16)
    x = rounded(2 * r.standard_normal((2, 2, 8, 96)), torch.bfloat16)
    g = rounded(r.standard_normal((2, 2, 8, 96)), torch.bfloat16)
    m = torch.zeros(2, 1, 1, 96, dtype=torch.float64)
    m[0, ..., 70:] = -10000.0
    keep = philox.keep_mask(x.numel(), 0.2, 31, 16).reshape(tuple(x.shape))
    y, dx, _ = chain(x, m, g, 0.125, keep=torch.from_numpy(keep.astype(np.float64)), p=0.2)
    out.update(drop_x=x.numpy(), drop_m=m.numpy(), drop_g=g.numpy(), drop_keep=keep, drop_out=y, drop_dx=dx)

    # inputs are exact in float32 (they hold bf16 / fp16 / fp32 values, the fills included)
    for key in list(out):
        if key.split("_")[1] in ("x", "m", "g"):
            assert np.array_equal(out[key].astype(np.float32).astype(np.float64), out[key]), key
            out[key] = out[key].astype(np.float32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "softmax_bias_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
