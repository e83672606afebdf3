"""Pins the optimizer steps of oracle/closed_form.py (SGD, Adagrad, NovoGrad, LAMB,
tensor norms) without a GPU: against torch.optim where torch has the algorithm,
and for the rest (NovoGrad, LAMB) against reductions to torch.optim.SGD /
torch.optim.Adam plus torch's vector norms, special cases that reduce to a
pinned routine, hand arithmetic on tiny inputs and invariants of the update."""
import numpy as np
import pytest
import torch

from oracle import closed_form as cf

# hyper-parameters exactly representable in float32 (the type the kernels, and so
# the oracle, receive them in): both sides then compute the same numbers
LR, WD, MU = 2.0 ** -5, 2.0 ** -4, 0.875


@pytest.mark.parametrize("momentum,dampening,nesterov", [(0.0, 0.0, False), (MU, 0.0, False),
                                                        (MU, 0.25, False), (MU, 0.0, True)])
@pytest.mark.parametrize("wd", [0.0, WD])
def test_sgd_step_vs_torch_optim(momentum, dampening, nesterov, wd):
    r = np.random.default_rng(1)
    w0 = r.standard_normal((4, 9))
    w_t = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.SGD([w_t], lr=LR, momentum=momentum, dampening=dampening, nesterov=nesterov,
                          weight_decay=wd)
    w, mom = w0.copy(), np.zeros_like(w0)
    for step in range(5):
        g = r.standard_normal((4, 9))
        w_t.grad = torch.from_numpy(g.copy())
        opt.step()
        w, mom, _ = cf.sgd_step(g, w, mom, LR, wd, momentum, dampening, nesterov, step == 0)
        assert np.allclose(w, w_t.detach().numpy(), rtol=1e-13, atol=1e-15), step
    if momentum:
        assert np.allclose(mom, opt.state[w_t]["momentum_buffer"].numpy(), rtol=1e-13)


def test_sgd_step_decay_order_scale_and_copy():
    r = np.random.default_rng(2)
    g, w, mom = r.standard_normal(50), r.standard_normal(50), r.standard_normal(50)
    # without momentum the place of the weight decay does not matter
    a = cf.sgd_step(g, w, mom, LR, WD, 0.0, 0.0, False, False, wd_after_momentum=False)
    b = cf.sgd_step(g, w, mom, LR, WD, 0.0, 0.0, False, False, wd_after_momentum=True)
    assert np.array_equal(a[0], b[0])
    assert np.array_equal(a[1], mom)  # and the buffer is left alone
    # with momentum: decay after the momentum step is w - lr * (mom' + wd * w) by hand
    c = cf.sgd_step(g, w, mom, LR, WD, MU, 0.0, False, False, wd_after_momentum=True)
    mom2 = MU * mom + g
    assert np.allclose(c[0], w - LR * (mom2 + WD * w), rtol=1e-14)
    assert np.allclose(c[1], mom2, rtol=1e-14)
    # scale multiplies the gradient first
    d = cf.sgd_step(4.0 * g, w, mom, LR, WD, MU, 0.0, False, False, scale=0.25)
    e = cf.sgd_step(g, w, mom, LR, WD, MU, 0.0, False, False)
    assert np.array_equal(d[0], e[0])
    # the 16-bit copy is a conversion of the stored float32 weight
    f = cf.sgd_step(g, w, mom, LR, 0.0, 0.0, 0.0, False, True, out="f32", copy="bf16")
    assert np.array_equal(f[2], cf.round_bf16(f[0]))
    assert f[0].dtype == np.float32 or np.array_equal(f[0], f[0].astype(np.float32))


@pytest.mark.parametrize("wd", [0.0, WD])
def test_adagrad_step_vs_torch_optim(wd):
    r = np.random.default_rng(3)
    p0 = r.standard_normal((6, 5))
    p_t = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    eps = 2.0 ** -20
    opt = torch.optim.Adagrad([p_t], lr=LR, eps=eps, weight_decay=wd)
    p, h = p0.copy(), np.zeros_like(p0)
    for step in range(5):
        g = r.standard_normal((6, 5))
        p_t.grad = torch.from_numpy(g.copy())
        opt.step()
        p, h = cf.adagrad_step(g, p, h, LR, eps, 0, wd)
        assert np.allclose(p, p_t.detach().numpy(), rtol=1e-13, atol=1e-15), step
    assert np.allclose(h, opt.state[p_t]["sum"].numpy(), rtol=1e-13)


def test_adagrad_decoupled_decay_by_hand():
    g, p, h = np.array([0.5, -2.0]), np.array([1.0, 3.0]), np.array([0.75, 5.0])
    p2, h2 = cf.adagrad_step(g, p, h, 0.5, 0.0, 1, 0.25)
    assert np.array_equal(h2, np.array([1.0, 9.0]))
    # p - lr * (g / sqrt(h') + decay * p)
    assert np.allclose(p2, np.array([1.0 - 0.5 * (0.5 / 1.0 + 0.25), 3.0 - 0.5 * (-2.0 / 3.0 + 0.75)]),
                       rtol=1e-15)
    # without decay the two modes coincide
    assert np.array_equal(cf.adagrad_step(g, p, h, 0.5, 1e-3, 0, 0.0)[0],
                          cf.adagrad_step(g, p, h, 0.5, 1e-3, 1, 0.0)[0])


def test_tensor_norms_vs_torch():
    r = np.random.default_rng(4)
    x = r.standard_normal(1000)
    assert np.isclose(cf.tensor_norm(x, 2), torch.linalg.vector_norm(torch.from_numpy(x)).item(), rtol=1e-14)
    assert cf.tensor_norm(x, 0) == np.abs(x).max()
    assert cf.tensor_norm(np.zeros(0)) == 0.0
    # blending: alpha = 0, beta = 1 gives the norm itself; the L2 blend is a norm of norms
    assert np.isclose(cf.blend_norm(7.0, x, 0.0, 1.0, 2), cf.tensor_norm(x, 2), rtol=1e-15)
    assert np.isclose(cf.blend_norm(3.0, np.array([4.0]), 1.0, 1.0, 2), 5.0, rtol=1e-15)
    assert np.isclose(cf.blend_norm(3.0, np.array([-4.0, 1.0]), 0.5, 0.25, 0), 2.5, rtol=1e-15)


def test_novograd_step_special_cases():
    r = np.random.default_rng(5)
    g, p, m = r.standard_normal(40), r.standard_normal(40), 0.1 * r.standard_normal(40)
    n = cf.tensor_norm(g)
    # beta1 = 0, no averaging, no decay, no bias correction: a normalised gradient step
    p2, m2 = cf.novograd_step(g, p, m, n, LR, 0.0, 0.5, 0.0, 1, False, 0.0, False, 1)
    assert np.allclose(p2, p - LR * g / n, rtol=1e-14) and np.allclose(m2, g, rtol=1e-15)
    assert np.isclose(np.linalg.norm(p2 - p), LR, rtol=1e-13)  # a step of length lr
    # mode 0 keeps the moment of the normalised gradient, mode 1 of the raw one:
    # without weight decay the two steps differ only in whether the old moment
    # is divided by the norm
    a = cf.novograd_step(g, p, m, n, LR, MU, 0.75, 2.0 ** -10, 3, True, 0.0, True, 0)
    b = cf.novograd_step(g, p, m, n, LR, MU, 0.75, 2.0 ** -10, 3, True, 0.0, True, 1)
    assert np.allclose(a[0] - p, b[0] - p + LR * MU * (m / n_denom(n, 0.75, 3) - m) / (1 - MU ** 3),
                       rtol=1e-9, atol=1e-12)
    # by hand, mode 1 with everything on
    bc1, bc2 = 1 - MU ** 3, np.sqrt(1 - 0.75 ** 3)
    m3 = MU * m + (1 - MU) * g
    want = p - LR * ((m3 / np.float32(bc1)) / (n / np.float32(bc2) + 2.0 ** -10) + WD * p)
    c = cf.novograd_step(g, p, m, n, LR, MU, 0.75, 2.0 ** -10, 3, True, WD, True, 1)
    assert np.allclose(c[0], want, rtol=1e-13) and np.allclose(c[1], m3, rtol=1e-15)


def n_denom(n, beta2, step):
    return n / np.float64(np.float32(np.sqrt(1 - beta2 ** step))) + 2.0 ** -10


def test_lamb_reduces_to_adam_without_decay():
    """Without weight decay (and without use_nvlamb) the trust ratio is lr, and
    with a gradient norm below the clip threshold LAMB is the Adam step that
    test_oracle_adam.py pins against torch.optim."""
    r = np.random.default_rng(6)
    g, p = r.standard_normal(64), r.standard_normal(64)
    m, v = 0.1 * r.standard_normal(64), np.abs(r.standard_normal(64))
    for mode in (0, 1):
        u, m2, v2 = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 4, True, 0.0, True, mode,
                                   cf.tensor_norm(g), 1e9)
        p2 = cf.lamb_stage2(u, p, cf.tensor_norm(p), cf.tensor_norm(u), LR, 0.0, False)
        pa, ma, va = cf.adam_step(g, p, m, v, LR, MU, 0.75, 2.0 ** -20, 4, mode, True, 0.0)
        assert np.allclose(p2, pa, rtol=1e-14) and np.array_equal(m2, ma) and np.array_equal(v2, va)


def test_lamb_trust_ratio_clip_and_modes():
    r = np.random.default_rng(7)
    g, p = r.standard_normal(64), r.standard_normal(64)
    m, v = 0.1 * r.standard_normal(64), np.abs(r.standard_normal(64))
    gn = cf.tensor_norm(g)
    u, _, _ = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, WD, True, 1, gn, 1e9)
    pn, un = cf.tensor_norm(p), cf.tensor_norm(u)
    p2 = cf.lamb_stage2(u, p, pn, un, LR, WD, False)
    # the step has length lr * |p| whatever the update's size
    assert np.isclose(np.linalg.norm(p2 - p), LR * pn, rtol=1e-13)
    # a zero norm switches the ratio off
    assert np.allclose(cf.lamb_stage2(u, p, 0.0, un, LR, WD, False), p - LR * u, rtol=1e-15)
    # use_nvlamb applies the ratio without decay as well
    assert np.allclose(cf.lamb_stage2(u, p, pn, un, LR, 0.0, True), p - LR * pn / un * u, rtol=1e-14)
    # clipping: a global norm of twice the threshold halves the gradient
    a = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, 0.0, True, 1, 2.0, 1.0)
    b = cf.lamb_stage1(0.5 * g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, 0.0, True, 1, 0.5, 1.0)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    # mode 0 feeds the decay through the moments, mode 1 adds it to the update
    l2 = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, WD, True, 0, gn, 1e9)
    same = cf.lamb_stage1(g + WD * p, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, 0.0, True, 1, gn, 1e9)
    assert all(np.allclose(x, y, rtol=1e-14) for x, y in zip(l2, same))
    dec = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, WD, True, 1, gn, 1e9)
    nodec = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, 0.0, True, 1, gn, 1e9)
    assert np.allclose(dec[0], nodec[0] + WD * p, rtol=1e-14)
    # no gradient averaging: beta3 = 1
    na = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, False, 0.0, False, 1, gn, 1e9)
    assert np.allclose(na[1], MU * m + g, rtol=1e-15)


def test_lamb_gradient_scale_and_update_type():
    """The mixed-precision variant multiplies the gradient by the inverse loss
    scale first and stores the update in the gradients' type."""
    r = np.random.default_rng(8)
    g, p = r.standard_normal(64), r.standard_normal(64)
    m, v = 0.1 * r.standard_normal(64), np.abs(r.standard_normal(64))
    a = cf.lamb_stage1(1024.0 * g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, WD, True, 1, 1.0, 1e9,
                       inv_scale=2.0 ** -10)
    b = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, WD, True, 1, 1.0, 1e9)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    c = cf.lamb_stage1(g, p, m, v, MU, 0.75, 2.0 ** -20, 2, True, WD, True, 1, 1.0, 1e9, out="f32",
                       out_update="bf16")
    assert np.array_equal(c[0], cf.round_bf16(b[0].astype(np.float32)))
    assert np.array_equal(c[1], b[1].astype(np.float32))


@pytest.mark.parametrize("moment_mode", [0, 1])
@pytest.mark.parametrize("grad_averaging", [True, False])
def test_novograd_is_momentum_sgd_on_the_normalised_gradient(moment_mode, grad_averaging):
    """NovoGrad keeps one second moment per tensor (a scalar), so its
    element-wise part is torch.optim.SGD with momentum: in mode 0 on the
    gradient g / (norm + eps) + decay * p with dampening beta1 (gradient
    averaging) or 0, in mode 1 on the raw gradient with the step divided by
    norm + eps and the decay applied to the old weight.  Five steps, the norm
    following blend_norm (pinned against torch.linalg.vector_norm above), no
    bias correction (its two scalars are pinned by hand above)."""
    r = np.random.default_rng(11)
    beta2, eps = 0.75, 2.0 ** -10
    p0 = r.standard_normal((5, 8))
    p_t = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    p, m, norm = p0.copy(), np.zeros_like(p0), 0.0
    buf = None
    for step in range(1, 6):
        g = r.standard_normal((5, 8))
        # the first step stores the plain norm, later ones blend (fused_novograd.py:199-207 of the reference)
        norm = float(torch.linalg.vector_norm(torch.from_numpy(g))) if step == 1 else float(
            np.sqrt(beta2 * norm ** 2 + (1 - beta2) * float(torch.linalg.vector_norm(torch.from_numpy(g))) ** 2))
        denom = norm + eps
        old = p_t.detach().clone()
        if moment_mode == 0:
            lr_t, grad = LR, torch.from_numpy(g) / denom + WD * old
        else:
            lr_t, grad = LR / denom, torch.from_numpy(g.copy())
        opt = torch.optim.SGD([p_t], lr=lr_t, momentum=MU, dampening=MU if grad_averaging else 0.0)
        # (a zero buffer instead of torch's first-step copy of the gradient: the kernel's moment starts at zero)
        opt.state[p_t]["momentum_buffer"] = torch.zeros_like(p_t) if buf is None else buf
        p_t.grad = grad
        opt.step()
        buf = opt.state[p_t]["momentum_buffer"]
        if moment_mode == 1:
            with torch.no_grad():
                p_t -= LR * WD * old
        p, m = cf.novograd_step(g, p, m, norm, LR, MU, beta2, eps, step, False, WD, grad_averaging, moment_mode)
        assert np.allclose(p, p_t.detach().numpy(), rtol=1e-12, atol=1e-14), step
        assert np.allclose(m, buf.numpy(), rtol=1e-12, atol=1e-14), step


@pytest.mark.parametrize("mode", [0, 1])
def test_lamb_is_the_adam_direction_under_a_trust_ratio(mode):
    """Five LAMB steps assembled from library pieces: torch.optim.Adam with
    lr = 1 and no decay gives the direction a = m_hat / (sqrt(v_hat) + eps) (on
    g + decay * p in mode 0), the update is u = a (+ decay * p in mode 1), and
    the weight moves by lr * |p| / |u| * u with torch's vector norms; the
    gradient is first divided by max(1, global norm / threshold)."""
    r = np.random.default_rng(12)
    beta2, eps, max_norm = 0.75, 2.0 ** -20, 4.0
    p0 = r.standard_normal((6, 7))
    shadow = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    adam = torch.optim.Adam([shadow], lr=1.0, betas=(MU, beta2), eps=eps, weight_decay=0.0)
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    p_t = torch.from_numpy(p0.copy())
    for step in range(1, 6):
        g = (3.0 if step % 2 else 0.3) * r.standard_normal((6, 7))   # some steps are clipped, some not
        gn = float(torch.linalg.vector_norm(torch.from_numpy(g)))
        clipped = torch.from_numpy(g) / max(1.0, gn / max_norm)
        with torch.no_grad():
            shadow.copy_(p_t)
        shadow.grad = clipped + WD * p_t if mode == 0 else clipped
        adam.step()
        a = p_t - shadow.detach()                       # the Adam direction (lr = 1)
        u = a + WD * p_t if mode == 1 else a
        ratio = LR * float(torch.linalg.vector_norm(p_t)) / float(torch.linalg.vector_norm(u))
        p_t = p_t - ratio * u
        upd, m, v = cf.lamb_stage1(g, p, m, v, MU, beta2, eps, step, True, WD, True, mode, gn, max_norm)
        assert np.allclose(upd, u.numpy(), rtol=1e-11, atol=1e-13), step
        p = cf.lamb_stage2(upd, p, cf.tensor_norm(p), cf.tensor_norm(upd), LR, WD, False)
        assert np.allclose(p, p_t.numpy(), rtol=1e-11, atol=1e-13), step
        st = adam.state[shadow]
        assert np.allclose(m, st["exp_avg"].numpy(), rtol=1e-12) and np.allclose(v, st["exp_avg_sq"].numpy(), rtol=1e-12)
