"""Pins oracle/closed_form.adam_step against torch's own CPU Adam / AdamW over
several steps in float64 (no GPU needed)."""
import numpy as np
import pytest
import torch

from oracle import closed_form as cf


@pytest.mark.parametrize("adamw", [False, True])
@pytest.mark.parametrize("bias_correction", [True])
@pytest.mark.parametrize("wd", [0.0, 0.0625])
def test_adam_step_vs_torch_optim(adamw, bias_correction, wd):
    r = np.random.default_rng(3)
    p0 = r.standard_normal((5, 7))
    p_t = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    cls = torch.optim.AdamW if adamw else torch.optim.Adam
    # hyper-parameters exactly representable in float32, the type the kernel (and
    # so the oracle) receives them in: then both sides compute the same numbers
    lr, b1, b2, eps = 2.0 ** -7, 0.875, 1.0 - 2.0 ** -10, 2.0 ** -27
    opt = cls([p_t], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    for step in range(1, 6):
        g = r.standard_normal((5, 7))
        p_t.grad = torch.from_numpy(g.copy())
        opt.step()
        p, m, v = cf.adam_step(g, p, m, v, lr, b1, b2, eps, step, 1 if adamw else 0,
                               bias_correction, wd)
        # (the oracle stores the bias corrections as float32, as the kernel does)
        assert np.allclose(p, p_t.detach().numpy(), rtol=1e-6, atol=1e-9), step
    st = opt.state[p_t]
    assert np.allclose(m, st["exp_avg"].numpy(), rtol=1e-12, atol=1e-15)
    assert np.allclose(v, st["exp_avg_sq"].numpy(), rtol=1e-12, atol=1e-15)


def test_adam_step_modes_differ_and_no_bias_correction():
    r = np.random.default_rng(4)
    g, p = r.standard_normal(100), r.standard_normal(100)
    m, v = 0.1 * r.standard_normal(100), np.abs(r.standard_normal(100))
    l2 = cf.adam_step(g, p, m, v, 1e-3, 0.9, 0.999, 1e-8, 3, 0, True, 0.1)
    aw = cf.adam_step(g, p, m, v, 1e-3, 0.9, 0.999, 1e-8, 3, 1, True, 0.1)
    assert not np.allclose(l2[0], aw[0], rtol=1e-9)
    assert not np.allclose(l2[1], aw[1], rtol=1e-9)  # L2 changes the moments, AdamW does not
    same = cf.adam_step(g, p, m, v, 1e-3, 0.9, 0.999, 1e-8, 3, 1, True, 0.0)
    assert np.array_equal(same[1], aw[1]) and np.array_equal(same[2], aw[2])
    # without bias correction: p - lr * m' / (sqrt(v') + eps) by hand
    nb = cf.adam_step(g, p, m, v, 1e-3, 0.9, 0.999, 1e-8, 3, 1, False, 0.0)
    b1, b2 = float(np.float32(0.9)), float(np.float32(0.999))
    m2 = b1 * m + (1 - b1) * g
    v2 = b2 * v + (1 - b2) * g * g
    want = p - float(np.float32(1e-3)) * m2 / (np.sqrt(v2) + float(np.float32(1e-8)))
    assert np.allclose(nb[0], want, rtol=1e-14)
