"""Multi-tensor SGD, Adagrad, NovoGrad, LAMB and the tensor norms on the GPU,
through the C ABI, against the float64 oracle (oracle/closed_form.py, pinned by
test_oracle_optimizers.py): fp32 to 1e-5 relative, 16-bit results against the
oracle rounded once to the storage type."""
import os

import numpy as np
import pytest
import torch

from helpers import NP_NAME, check, f64, randn
from oracle import closed_form as cf
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

# lengths around the vector and piece boundaries of every dtype, an empty tensor,
# and more tensors than one launch carries (48)
SIZES = [1, 7, 4096, 4097, 8191, 8192, 100003, 3, 1 << 19, 0, 12345] + [257 + i for i in range(45)]
CHECKED = [0, 1, 2, 3, 4, 5, 6, 7, 8, 10, 11, 47, 48, 49, 55]


def make_lists(dtypes, seed, device, positive=()):
    host = []
    for k, dt in enumerate(dtypes):
        lst = []
        for i, n in enumerate(SIZES):
            t = randn((n,), dt, seed + 1000 * k + i, std=0.1 if k in positive else 1.0)
            lst.append(t.abs() if k in positive else t)
        host.append(lst)
    return host, [[t.to(device) for t in lst] for lst in host]


# 16-bit: the fp32 evaluation (several roundings before the store) lands on the
# other side of a rounding tie slightly more often than 0.2 % of the time; and a
# final multiply-add may be rounded to float16 once instead of twice
def kw(dtype):
    return {} if dtype == F32 else {"min_exact": 0.99, "single_rounding_too": True}


def unrounded(dtype):
    """The oracle's `out` for a check: 16-bit results are compared from the
    unrounded float64 value, so that either rounding can be recognised."""
    return "f64" if dtype != F32 else "f32"


@pytest.mark.parametrize("gdtype,wdtype,copy", [(F32, F32, None), (F16, F16, None), (BF16, BF16, None),
                                                (F16, F32, F16), (BF16, F32, BF16), (F32, F32, BF16),
                                                (BF16, F32, None), (F16, F32, None), (F16, F32, BF16),
                                                (BF16, F32, F16), (F32, F32, F16)])
@pytest.mark.parametrize("momentum,dampening,nesterov,wd,after", [
    (0.0, 0.0, False, 0.0, False), (0.9, 0.0, False, 0.01, False), (0.9, 0.1, False, 0.01, True),
    (0.9, 0.0, True, 0.01, False)])
def test_multi_tensor_sgd_vs_oracle(device, gdtype, wdtype, copy, momentum, dampening, nesterov, wd, after):
    dts = [gdtype, wdtype, wdtype] + ([copy] if copy else [])
    host, devl = make_lists(dts, 20, device)
    k = _C.get_sgd_kernel()
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    lr, scale = 0.05, 0.5
    want_w = [f64(t) for t in host[1]]
    want_m = [f64(t) for t in host[2]]
    for step in range(3):
        k.multi_tensor_sgd(2048 * 32, flag, devl, wd, momentum, dampening, lr, nesterov, step == 0, after, scale)
        for i in CHECKED:
            w, m, c = cf.sgd_step(f64(host[0][i]), want_w[i], want_m[i], lr, wd, momentum, dampening,
                                  nesterov, step == 0, after, scale, out=unrounded(wdtype),
                                  copy=NP_NAME[copy] if copy else None)
            what = "tensor %d step %d" % (i, step)
            if SIZES[i]:
                check(devl[1][i], w, "w " + what, atol=1e-6, **kw(wdtype))
                if momentum:
                    # 0.9 mom + 0.9 g of two 16-bit values lies within 3e-8 (relative) of
                    # a rounding tie for about one value in ten -- float32(0.9) is that
                    # far from 0.9 -- which is the resolution of the float32 evaluation
                    # itself: which neighbour is stored then depends on the order of the
                    # float32 operations (never more than 1 ulp apart)
                    loose = dict(kw(wdtype), min_exact=0.95) if wdtype != F32 else {}
                    check(devl[2][i], m, "mom " + what, atol=1e-6, **loose)
                else:
                    assert torch.equal(devl[2][i].cpu(), host[2][i]), "momentum buffer written"
                if copy:
                    # the copy is a conversion of the weight the kernel stored
                    assert torch.equal(devl[3][i], devl[1][i].to(copy)), "copy " + what
            want_w[i], want_m[i] = f64(devl[1][i]), f64(devl[2][i])
    for i in CHECKED:
        assert torch.equal(devl[0][i].cpu(), host[0][i]), "gradients must not change"
    # a raised flag switches the whole launch off
    before = [t.clone() for t in devl[1]]
    flag.fill_(1)
    k.multi_tensor_sgd(2048 * 32, flag, devl, wd, momentum, dampening, lr, nesterov, False, after, scale)
    assert all(torch.equal(a, b) for a, b in zip(before, devl[1]))


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("mode,wd", [(0, 0.0), (0, 0.01), (1, 0.01)])
def test_multi_tensor_adagrad_vs_oracle(device, dtype, mode, wd):
    host, devl = make_lists([dtype] * 3, 30, device, positive=(2,))
    k = _C.get_adagrad_kernel()
    lr, eps = 0.05, 1e-10
    want_p = [f64(t) for t in host[1]]
    want_h = [f64(t) for t in host[2]]
    for step in range(3):
        k.multi_tensor_adagrad(2048 * 32, None, devl, lr, eps, mode, wd)
        for i in CHECKED:
            p, h = cf.adagrad_step(f64(host[0][i]), want_p[i], want_h[i], lr, eps, mode, wd, out=unrounded(dtype))
            if SIZES[i]:
                check(devl[1][i], p, "p[%d] step %d" % (i, step), atol=1e-6, **kw(dtype))
                check(devl[2][i], h, "h[%d] step %d" % (i, step), atol=1e-7, **kw(dtype))
            want_p[i], want_h[i] = f64(devl[1][i]), f64(devl[2][i])


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_multi_tensor_l2norm(device, dtype):
    host, devl = make_lists([dtype], 40, device)
    k = _C.get_l2norm_kernel()
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    total, per = k.multi_tensor_l2norm(2048 * 32, flag, devl, True)
    want = np.array([cf.tensor_norm(f64(t)) for t in host[0]])
    assert per.dtype == torch.float32 and per.shape == (len(SIZES),)
    assert np.allclose(f64(per), want, rtol=2e-6, atol=0.0)
    assert np.isclose(f64(total)[0], np.sqrt((want ** 2).sum()), rtol=2e-6)
    assert per[SIZES.index(0)].item() == 0.0
    assert flag.item() == 0
    total2, per2 = k.multi_tensor_l2norm(2048 * 32, flag, devl, False)
    assert per2.numel() == 0 and torch.equal(total2, total)  # a fixed summation order
    # unaligned views take the scalar path
    base = randn((5000,), dtype, 41).to(device)
    views = [base[1:1001], base[1003:4000]]
    _, pv = k.multi_tensor_l2norm(0, None, [views], True)
    assert np.allclose(f64(pv), [cf.tensor_norm(f64(v)) for v in views], rtol=2e-6)
    # a value that is not finite reaches the result and raises the flag
    devl[0][4][17] = float("inf")
    total3, _ = k.multi_tensor_l2norm(2048 * 32, flag, devl, False)
    assert torch.isinf(total3).all() and flag.item() == 1


def test_largest_magnitude_over_all_tensors(device):
    """norm_type 0 with a result over all tensors (the C entry point takes it;
    the reference's bindings only ask for it per tensor)."""
    host, devl = make_lists([F16], 60, device)
    k = _C.get_l2norm_kernel()
    total = torch.empty(1, dtype=torch.float32, device=device)
    per = torch.empty(len(SIZES), dtype=torch.float32, device=device)
    k._run(devl[0], total, per, 0, 0, 0.0, 0.0, None)
    want = [float(np.abs(f64(t)).max()) if t.numel() else 0.0 for t in host[0]]
    assert np.array_equal(f64(per), np.array(want)) and total.item() == max(want)


@pytest.mark.parametrize("norm_type", [2, 0])
def test_multi_tensor_norm_out_blends(device, norm_type):
    host, devl = make_lists([BF16], 50, device)
    k = _C.get_l2norm_kernel()
    g = torch.Generator().manual_seed(5)
    old = torch.rand(len(SIZES), generator=g) + 0.5
    out = old.to(device)
    k.multi_tensor_norm_out(2048 * 32, None, devl, out, 0.75, 0.25, norm_type)
    want = [cf.blend_norm(old[i].item(), f64(t), 0.75, 0.25, norm_type) for i, t in enumerate(host[0])]
    assert np.allclose(f64(out), want, rtol=2e-6)


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("moment_mode,wd,averaging,norm_type", [(1, 0.0, 1, 2), (0, 0.01, 1, 2), (1, 0.01, 0, 0)])
def test_multi_tensor_novograd_vs_oracle(device, dtype, moment_mode, wd, averaging, norm_type):
    host, devl = make_lists([dtype] * 3, 60, device)
    k = _C.get_novograd_kernel()
    lr, b1, b2, eps = 0.01, 0.95, 0.98, 1e-8
    norms0 = torch.tensor([float(cf.tensor_norm(f64(t), norm_type)) for t in host[0]], dtype=torch.float32)
    norms = norms0.to(device)
    want_p = [f64(t) for t in host[1]]
    want_m = [f64(t) for t in host[2]]
    want_n = [float(v) for v in norms0]
    for step in (1, 2, 5):
        k.multi_tensor_novograd(2048 * 32, None, devl, norms, lr, b1, b2, eps, step, 1, wd, averaging,
                                moment_mode, norm_type)
        got_n = f64(norms)
        for i in CHECKED:
            n = cf.blend_norm(want_n[i], f64(host[0][i]), b2, 1.0 - b2, norm_type)
            assert np.isclose(got_n[i], n, rtol=2e-6), "norm %d step %d" % (i, step)
            # the element-wise step from the norm the kernel stored
            p, m = cf.novograd_step(f64(host[0][i]), want_p[i], want_m[i], got_n[i], lr, b1, b2, eps, step,
                                    True, wd, averaging, moment_mode, out=unrounded(dtype))
            if SIZES[i]:
                check(devl[1][i], p, "p[%d] step %d" % (i, step), atol=1e-6, **kw(dtype))
                check(devl[2][i], m, "m[%d] step %d" % (i, step), atol=1e-6, **kw(dtype))
            want_p[i], want_m[i], want_n[i] = f64(devl[1][i]), f64(devl[2][i]), got_n[i]


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("mode,wd,nvlamb,clip", [(1, 0.01, False, 1e9), (0, 0.01, False, 1e9),
                                                 (1, 0.0, False, 1e9), (1, 0.0, True, 1.0)])
def test_multi_tensor_lamb_vs_oracle(device, dtype, mode, wd, nvlamb, clip):
    host, devl = make_lists([dtype] * 4, 70, device, positive=(3,))
    k = _C.get_lamb_kernel()
    lr, b1, b2, eps, step = 0.01, 0.9, 0.999, 1e-6, 3
    gn = float(np.sqrt(sum(cf.tensor_norm(f64(t)) ** 2 for t in host[0])))
    gnorm = torch.tensor([gn], dtype=torch.float32, device=device)
    k.multi_tensor_lamb(2048 * 32, None, devl, lr, b1, b2, eps, step, 1, wd, 1, mode, gnorm, clip, nvlamb)
    for i in CHECKED:
        if not SIZES[i]:
            continue
        u, m, v = cf.lamb_stage1(f64(host[0][i]), f64(host[1][i]), f64(host[2][i]), f64(host[3][i]), b1, b2, eps,
                                 step, True, wd, True, mode, np.float32(gn), clip, out=unrounded(dtype))
        what = "tensor %d" % i
        check(devl[0][i], u, "update " + what, atol=1e-6, **kw(dtype))
        check(devl[2][i], m, "m " + what, atol=1e-7, **kw(dtype))
        check(devl[3][i], v, "v " + what, atol=1e-8, **kw(dtype))
        # stage 2 from the update the kernel stored (its norm is what stage 2 saw)
        ud = f64(devl[0][i])
        p = cf.lamb_stage2(ud, f64(host[1][i]), np.float32(cf.tensor_norm(f64(host[1][i]))),
                           np.float32(cf.tensor_norm(ud)), lr, wd, nvlamb, out=unrounded(dtype))
        check(devl[1][i], p, "p " + what, atol=1e-6, **kw(dtype))


def test_argument_checks(device):
    a = torch.zeros(8, device=device)
    h = a.half()
    with pytest.raises(RuntimeError):
        _C.get_sgd_kernel().multi_tensor_sgd(0, None, [[a], [a]], 0, 0, 0, 0.1, False, True, False, 1.0)
    with pytest.raises(RuntimeError):  # float32 gradients with 16-bit weights
        _C.get_sgd_kernel().multi_tensor_sgd(0, None, [[a], [h], [h]], 0, 0, 0, 0.1, False, True, False, 1.0)
    with pytest.raises(RuntimeError):  # a copy of 16-bit weights
        _C.get_sgd_kernel().multi_tensor_sgd(0, None, [[h], [h], [h], [h]], 0, 0, 0, 0.1, False, True, False, 1.0)
    with pytest.raises(RuntimeError):  # momentum of another dtype than the weights
        _C.get_sgd_kernel().multi_tensor_sgd(0, None, [[h], [a], [h]], 0, 0, 0, 0.1, False, True, False, 1.0)
    with pytest.raises(RuntimeError):
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, None, [[a], [a], [a]], 0.1, 1e-10, 2, 0.0)
    with pytest.raises(RuntimeError):
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, None, [[a], [a, a], [a]], 0.1, 1e-10, 0, 0.0)
    with pytest.raises(RuntimeError):
        _C.get_l2norm_kernel().multi_tensor_norm_out(0, None, [[a]], torch.zeros(2, device=device), 0.5, 0.5, 2)
    with pytest.raises(RuntimeError):
        _C.get_l2norm_kernel().multi_tensor_norm_out(0, None, [[a]], torch.zeros(1, device=device), 0.5, 0.5, 1)
    with pytest.raises(RuntimeError):  # the flag must live on the GPU
        _C.get_l2norm_kernel().multi_tensor_l2norm(0, torch.zeros(1, dtype=torch.int32), [[a]], False)
    _C.get_adagrad_kernel().multi_tensor_adagrad(0, None, [[], [], []], 0.1, 1e-10, 0, 0.0)


# ---------------------------------------------------------------------------
# the optimizer classes
# ---------------------------------------------------------------------------
def _mlp(device):
    torch.manual_seed(0)
    return torch.nn.Sequential(
        torch.nn.Linear(64, 96), torch.nn.GELU(), torch.nn.Linear(96, 33), torch.nn.LayerNorm(33)
    ).to(device)


def _train(models_and_optimizers, device, steps=8, shared_gradients=False):
    """`shared_gradients`: every model steps on the gradients of the last one.
    An optimizer that normalises each element's step (Adagrad) turns a
    last-place difference in a near-zero gradient into a step of another size,
    so two trajectories on their own gradients drift apart for reasons that say
    nothing about the update rule."""
    g = torch.Generator(device=device).manual_seed(1)
    for _ in range(steps):
        x = torch.randn(16, 64, generator=g, device=device)
        for mdl, opt in models_and_optimizers:
            opt.zero_grad()
            mdl(x).square().mean().backward()
        if shared_gradients:
            src = list(models_and_optimizers[-1][0].parameters())
            for mdl, _ in models_and_optimizers[:-1]:
                for p, q in zip(mdl.parameters(), src):
                    p.grad = q.grad.clone()
        for _, opt in models_and_optimizers:
            opt.step()


@pytest.mark.parametrize("kwargs", [dict(), dict(momentum=0.9), dict(momentum=0.9, weight_decay=0.02),
                                    dict(momentum=0.9, nesterov=True), dict(momentum=0.8, dampening=0.2)])
def test_fused_sgd_tracks_torch_optim(device, kwargs):
    from oslo_amd.torch.optim import FusedSGD

    a, b = _mlp(device), _mlp(device)
    oa = FusedSGD(a.parameters(), lr=0.05, **kwargs)
    ob = torch.optim.SGD(b.parameters(), lr=0.05, **kwargs)
    _train([(a, oa), (b, ob)], device)
    for pa, pb in zip(a.parameters(), b.parameters()):
        assert torch.allclose(pa, pb, rtol=1e-5, atol=1e-6)
    if kwargs.get("momentum"):
        for pa, pb in zip(a.parameters(), b.parameters()):
            assert torch.allclose(oa.state[pa]["momentum_buffer"], ob.state[pb]["momentum_buffer"],
                                  rtol=1e-5, atol=1e-7)
    if not kwargs.get("momentum"):
        assert all("momentum_buffer" not in oa.state[p] for p in a.parameters())  # nothing allocated
    with pytest.raises(ValueError):
        FusedSGD(a.parameters(), lr=0.1, nesterov=True)
    with pytest.raises(ValueError):
        FusedSGD(a.parameters(), lr=-1.0)
    oa.zero_grad()
    assert all(p.grad is not None for p in a.parameters())  # set_grad_none defaults to False here


def test_fused_sgd_parameter_added_later_and_bf16(device):
    """A parameter that joins after the first step starts its momentum buffer on
    its own first step; bfloat16 and float32 parameters share a group."""
    from oslo_amd.torch.optim import FusedSGD

    p1 = torch.nn.Parameter(randn((300,), F32, 1).to(device))
    p2 = torch.nn.Parameter(randn((500,), BF16, 2).to(device))
    opt = FusedSGD([p1], lr=0.1, momentum=0.9)
    g1, g2 = randn((300,), F32, 3).to(device), randn((500,), BF16, 4).to(device)
    p1.grad = g1.clone()
    opt.step()
    opt.add_param_group({"params": [p2]})
    w1, w2 = f64(p1), f64(p2)
    m1 = f64(opt.state[p1]["momentum_buffer"])
    p1.grad, p2.grad = g1.clone(), g2.clone()
    opt.step()
    want1, wm1, _ = cf.sgd_step(f64(g1), w1, m1, 0.1, 0.0, 0.9, 0.0, False, False, out="f32")
    want2, wm2, _ = cf.sgd_step(f64(g2), w2, np.zeros(500), 0.1, 0.0, 0.9, 0.0, False, True, out="f64")
    check(p1.data, want1, "float32 parameter, second step")
    check(p2.data, want2, "bfloat16 parameter, first step", **kw(BF16))
    check(opt.state[p2]["momentum_buffer"], wm2, "its momentum buffer", **kw(BF16))


@pytest.mark.parametrize("wd", [0.0, 0.02])
def test_fused_adagrad_tracks_torch_optim(device, wd):
    from oslo_amd.torch.optim import FusedAdagrad

    a, b = _mlp(device), _mlp(device)
    oa = FusedAdagrad(a.parameters(), lr=0.05, weight_decay=wd)
    ob = torch.optim.Adagrad(b.parameters(), lr=0.05, weight_decay=wd, eps=1e-10)
    _train([(a, oa), (b, ob)], device, shared_gradients=True)
    for pa, pb in zip(a.parameters(), b.parameters()):
        assert torch.allclose(pa, pb, rtol=1e-5, atol=1e-6)
        assert torch.allclose(oa.state[pa]["sum"], ob.state[pb]["sum"], rtol=1e-5, atol=1e-12)
    oa.zero_grad()
    assert all(p.grad is None for p in a.parameters())


def _param_set(device, dtype):
    shapes = [(40, 30), (30,), (7, 5, 11)]
    ps = [torch.nn.Parameter(randn(s, dtype, 80 + i).to(device)) for i, s in enumerate(shapes)]
    grads = [[randn(s, dtype, 90 + 10 * step + i) for i, s in enumerate(shapes)] for step in range(4)]
    return ps, grads


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("init_zero,reg_inside,norm_type", [(False, False, 2), (True, True, 2), (False, False, 0)])
def test_fused_novograd_follows_the_oracle(device, dtype, init_zero, reg_inside, norm_type):
    from oslo_amd.torch.optim import FusedNovograd

    ps, grads = _param_set(device, dtype)
    lr, betas, eps, wd = 0.01, (0.95, 0.98), 1e-8, 0.01
    opt = FusedNovograd(ps, lr=lr, betas=betas, eps=eps, weight_decay=wd, init_zero=init_zero,
                        reg_inside_moment=reg_inside, norm_type=norm_type)
    want_p = [f64(p) for p in ps]
    want_m = [np.zeros(p.shape) for p in ps]
    want_n = [None] * len(ps)
    for step, gs in enumerate(grads, start=1):
        for p, g in zip(ps, gs):
            p.grad = g.to(device)
        opt.step()
        for i, g in enumerate(gs):
            if want_n[i] is None:
                want_n[i] = 0.0 if init_zero else float(cf.tensor_norm(f64(g), norm_type))
            want_n[i] = float(cf.blend_norm(want_n[i], f64(g), betas[1], 1.0 - betas[1], norm_type))
            p, m = cf.novograd_step(f64(g), want_p[i], want_m[i], np.float32(want_n[i]), lr, betas[0], betas[1],
                                    eps, step, True, wd, True, 0 if reg_inside else 1, out=unrounded(dtype))
            check(ps[i].data, p, "p[%d] step %d" % (i, step), atol=1e-6, **kw(dtype))
            want_p[i], want_m[i] = f64(ps[i]), f64(opt.state[ps[i]]["exp_avg"])
    assert opt.param_groups[0]["step"] == len(grads)
    with pytest.raises(RuntimeError):
        FusedNovograd(ps, amsgrad=True)
    with pytest.raises(RuntimeError):
        FusedNovograd(ps, norm_type=1)


@pytest.mark.parametrize("dtype", [F32, F16])
def test_fused_novograd_state_dict_round_trip_and_reference_layout(device, dtype):
    """The per-tensor norms live in the parameter group under plain string
    keys; a state dict written by the reference (a two-element list, norms of
    the 16-bit tensors then of the float32 tensors, oslo/torch/optim/
    fused_novograd.py:172-226) is accepted too.  Both continue the trajectory
    of an optimizer that was never saved."""
    import copy

    from oslo_amd.torch.optim import FusedNovograd

    def fresh():
        ps, grads = _param_set(device, dtype)
        return ps, grads, FusedNovograd(ps, lr=0.01, betas=(0.95, 0.98), weight_decay=0.01)

    def run(ps, grads, opt, steps):
        for gs in steps:
            for p, g in zip(ps, gs):
                p.grad = g.to(device)
            opt.step()

    ps, grads, opt = fresh()
    run(ps, grads, opt, grads)                       # never saved
    want = [p.detach().clone() for p in ps]
    for layout in ("own", "reference"):
        ps2, grads2, opt2 = fresh()
        run(ps2, grads2, opt2, grads2[:1])
        sd = copy.deepcopy(opt2.state_dict())
        norms = sd["param_groups"][0]["exp_avg_sq"]
        assert list(norms) == [str(dtype).split(".")[-1]]
        if layout == "reference":
            v = norms[str(dtype).split(".")[-1]]
            empty = torch.zeros(0, device=device)
            sd["param_groups"][0]["exp_avg_sq"] = [empty, v] if dtype == F32 else [v, empty]
        ps3, grads3, opt3 = fresh()
        with torch.no_grad():
            for a, b in zip(ps3, ps2):
                a.copy_(b)
        opt3.load_state_dict(sd)
        run(ps3, grads3, opt3, grads3[1:])
        for a, b in zip(ps3, want):
            assert torch.equal(a, b), layout


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("wd,max_grad_norm,nvlamb", [(0.01, 0.0, False), (0.0, 0.5, False), (0.0, 0.0, True)])
def test_fused_lamb_follows_the_oracle(device, dtype, wd, max_grad_norm, nvlamb):
    from oslo_amd.torch.optim import FusedLamb

    ps, grads = _param_set(device, dtype)
    lr, betas, eps = 0.01, (0.9, 0.999), 1e-6
    opt = FusedLamb(ps, lr=lr, betas=betas, eps=eps, weight_decay=wd, max_grad_norm=max_grad_norm,
                    use_nvlamb=nvlamb)
    want_p = [f64(p) for p in ps]
    want_m = [np.zeros(p.shape) for p in ps]
    want_v = [np.zeros(p.shape) for p in ps]
    for step, gs in enumerate(grads, start=1):
        for p, g in zip(ps, gs):
            p.grad = g.to(device)
        opt.step()
        gn = np.float32(np.sqrt(sum(cf.tensor_norm(f64(g)) ** 2 for g in gs)))
        clip = max_grad_norm if max_grad_norm > 0 else float("inf")
        for i, g in enumerate(gs):
            u, m, v = cf.lamb_stage1(f64(g), want_p[i], want_m[i], want_v[i], betas[0], betas[1], eps, step, True,
                                     wd, True, 1, gn, clip, out=unrounded(dtype))
            # the update direction is what the step left in the gradient; stage 2 started from it
            check(ps[i].grad, u, "update[%d] step %d" % (i, step), atol=1e-6, **kw(dtype))
            ud = f64(ps[i].grad)
            p = cf.lamb_stage2(ud, want_p[i], np.float32(cf.tensor_norm(want_p[i])), np.float32(cf.tensor_norm(ud)),
                               lr, wd, nvlamb, out=unrounded(dtype))
            check(ps[i].data, p, "p[%d] step %d" % (i, step), atol=2e-6, **kw(dtype))
            want_p[i] = f64(ps[i])
            want_m[i], want_v[i] = f64(opt.state[ps[i]]["exp_avg"]), f64(opt.state[ps[i]]["exp_avg_sq"])
    with pytest.raises(RuntimeError):
        FusedLamb(ps, amsgrad=True)
    with pytest.raises(RuntimeError):
        FusedLamb(ps, max_coeff=5.0)


# ---------------------------------------------------------------------------
# LAMB with device-resident scalars, an overflow flag and float32 master weights
# ---------------------------------------------------------------------------
def _scalars(device, lr, step, max_norm, inv_scale):
    f = lambda v, dt=torch.float32: torch.tensor([v], dtype=dt, device=device)
    return f(lr), f(step, torch.int32), f(max_norm), f(inv_scale)


@pytest.mark.parametrize("gdtype,master", [(F32, False), (BF16, False), (F16, True), (BF16, True), (F16, False),
                                           (F32, True)])
@pytest.mark.parametrize("mode,wd,nvlamb", [(1, 0.01, False), (0, 0.01, False), (1, 0.0, True)])
def test_multi_tensor_lamb_mp_vs_oracle(device, gdtype, master, mode, wd, nvlamb):
    pdtype = F32 if master else gdtype
    dts = [gdtype, pdtype, pdtype, pdtype] + ([gdtype] if master else [])
    host, devl = make_lists(dts, 110, device, positive=(3,))
    k = _C.get_lamb_mp_kernel()
    b1, b2, eps, step, scale = 0.9, 0.999, 1e-6, 3, 256.0
    lr, step_t, max_norm, inv_scale = _scalars(device, 0.01, step, 1.0 * scale, 1.0 / scale)
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    # the gradients arrive multiplied by the loss scale; so does their norm
    gn = np.float32(np.sqrt(sum(cf.tensor_norm(f64(t)) ** 2 for t in host[0])))
    gnorm = torch.tensor([gn], dtype=torch.float32, device=device)
    found_inf = torch.zeros(1, device=device)
    k.multi_tensor_lamb_mp(0, flag, devl, lr, b1, b2, eps, step_t, 1, wd, 1, mode, gnorm, max_norm, nvlamb,
                           found_inf, inv_scale)
    assert flag.item() == 0
    for i in CHECKED:
        if not SIZES[i]:
            continue
        u, m, v = cf.lamb_stage1(f64(host[0][i]), f64(host[1][i]), f64(host[2][i]), f64(host[3][i]), b1, b2, eps,
                                 step, True, wd, True, mode, gn, 1.0 * scale, out=unrounded(pdtype),
                                 inv_scale=1.0 / scale, out_update=unrounded(gdtype))
        what = "tensor %d" % i
        check(devl[0][i], u, "update " + what, atol=1e-6, **kw(gdtype))
        check(devl[2][i], m, "m " + what, atol=1e-7, **kw(pdtype))
        check(devl[3][i], v, "v " + what, atol=1e-8, **kw(pdtype))
        ud = f64(devl[0][i])
        p = cf.lamb_stage2(ud, f64(host[1][i]), np.float32(cf.tensor_norm(f64(host[1][i]))),
                           np.float32(cf.tensor_norm(ud)), 0.01, wd, nvlamb, out=unrounded(pdtype))
        check(devl[1][i], p, "p " + what, atol=1e-6, **kw(pdtype))
        if master:
            assert torch.equal(devl[4][i], devl[1][i].to(gdtype)), "model copy " + what
    # while the flag is raised nothing is touched, not even the gradients
    before = [[t.clone() for t in lst] for lst in devl]
    flag.fill_(1)
    k.multi_tensor_lamb_mp(0, flag, devl, lr, b1, b2, eps, step_t, 1, wd, 1, mode, gnorm, max_norm, nvlamb,
                           found_inf, inv_scale)
    for la, lb in zip(before, devl):
        assert all(torch.equal(a, b) for a, b in zip(la, lb))


def test_l2norm_mp_skips_while_the_flag_is_raised(device):
    k = _C.get_l2norm_mp_kernel()
    xs = [randn((5000,), F32, 1).to(device), randn((300,), F32, 2).to(device)]
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    total, per = k.multi_tensor_l2norm_mp(0, flag, [xs], True)
    want = [cf.tensor_norm(f64(x)) for x in xs]
    assert np.allclose(f64(per), want, rtol=2e-6) and np.isclose(total.item(), np.hypot(*want), rtol=2e-6)
    # a non-finite value raises the flag; the next call leaves its outputs alone
    xs[0][7] = float("nan")
    k.multi_tensor_l2norm_mp(0, flag, [xs], True)
    assert flag.item() == 1
    lib = _C.load_library()
    import ctypes
    out = torch.full((2,), -7.0, device=device)
    glob = torch.full((1,), -7.0, device=device)
    part = torch.zeros(8, device=device)
    arr = (ctypes.c_void_p * 2)(*[x.data_ptr() for x in xs])
    sizes = (ctypes.c_int64 * 2)(5000, 300)
    rc = lib.oslo_multi_tensor_norm(arr, sizes, 2, 0, part.data_ptr(), 8, glob.data_ptr(), out.data_ptr(), 2, 0,
                                    0.0, 0.0, flag.data_ptr(), 1, torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and (out == -7.0).all() and glob.item() == -7.0
    with pytest.raises(RuntimeError):
        k.multi_tensor_l2norm_mp(0, None, [xs], True)


@pytest.mark.parametrize("reduced", [None, BF16])
def test_fused_mixed_precision_lamb_follows_the_oracle(device, reduced):
    from oslo_amd.torch.optim import FusedMixedPrecisionLamb

    dtype = reduced or F32
    ps, grads = _param_set(device, dtype)
    lr, betas, eps, wd, clip = 0.01, (0.9, 0.999), 1e-6, 0.01, 0.5
    opt = FusedMixedPrecisionLamb(ps, lr=lr, betas=betas, eps=eps, weight_decay=wd, max_grad_norm=clip,
                                  reduced_precision_dtype=reduced)
    want_p = [f64(p) for p in ps]
    want_m = [np.zeros(p.shape) for p in ps]
    want_v = [np.zeros(p.shape) for p in ps]
    for step, gs in enumerate(grads, start=1):
        for p, g in zip(ps, gs):
            p.grad = g.to(device)
        opt.step()
        gn = np.float32(np.sqrt(sum(cf.tensor_norm(f64(g)) ** 2 for g in gs)))
        for i, g in enumerate(gs):
            u, m, v = cf.lamb_stage1(f64(g), want_p[i], want_m[i], want_v[i], betas[0], betas[1], eps, step, True,
                                     wd, True, 1, gn, clip, out="f32", out_update=unrounded(dtype))
            # the update direction is what the step left in the gradient; stage 2 started from it
            check(ps[i].grad, u, "update[%d] step %d" % (i, step), atol=1e-6, **kw(dtype))
            ud = f64(ps[i].grad)
            p = cf.lamb_stage2(ud, want_p[i], np.float32(cf.tensor_norm(want_p[i])), np.float32(cf.tensor_norm(ud)),
                               lr, wd, False, out="f32")
            full = opt.param_groups_full_precision[0]["params"][i]
            held = full if reduced else ps[i].data
            check(held, p, "p[%d] step %d" % (i, step), atol=2e-6)
            if reduced:
                assert full.dtype == F32 and torch.equal(ps[i].data, full.to(reduced))
                assert opt.state[ps[i]]["exp_avg"].dtype == F32
            want_p[i] = f64(held)
            want_m[i], want_v[i] = f64(opt.state[ps[i]]["exp_avg"]), f64(opt.state[ps[i]]["exp_avg_sq"])
    assert opt.param_groups[0]["step"].item() == len(grads) and opt.param_groups[0]["step"].is_cuda
    # the state survives a round trip without being cast to the parameters' dtype
    sd = opt.state_dict()
    opt.load_state_dict(sd)
    assert opt.state[ps[0]]["exp_avg"].dtype == (F32 if reduced else dtype)


def test_fused_mixed_precision_lamb_with_a_grad_scaler(device):
    """Through torch.amp.GradScaler: scaled gradients give the unscaled step, and
    a step whose gradients overflow changes nothing and is not counted."""
    from oslo_amd.torch.optim import FusedMixedPrecisionLamb

    def run(scaled):
        torch.manual_seed(0)
        model = torch.nn.Linear(48, 32).to(device)
        opt = FusedMixedPrecisionLamb(model.parameters(), lr=0.01)
        scaler = torch.amp.GradScaler("cuda", init_scale=1024.0, enabled=scaled)
        g = torch.Generator(device=device).manual_seed(1)
        for _ in range(3):
            x = torch.randn(8, 48, generator=g, device=device)
            opt.zero_grad()
            scaler.scale(model(x).square().mean()).backward()
            scaler.step(opt)
            scaler.update()
        return model, opt, scaler

    plain, _, _ = run(False)
    model, opt, scaler = run(True)
    for a, b in zip(plain.parameters(), model.parameters()):
        assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)
    before = [p.detach().clone() for p in model.parameters()]
    opt.zero_grad()
    scaler.scale(model(torch.full((8, 48), float("inf"), device=device)).square().mean()).backward()
    scaler.step(opt)
    scaler.update()
    assert all(torch.equal(a, b) for a, b in zip(before, model.parameters()))
    assert opt.param_groups[0]["step"].item() == 3 and scaler.get_scale() == 512.0


# ---------------------------------------------------------------------------
# random lists: tensor counts across the launch boundary, lengths around every
# piece boundary, views at odd offsets of one buffer, every step and dtype
# ---------------------------------------------------------------------------
def _random_cases(count, seed):
    r = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        nt = int(r.choice([1, 2, 5, 47, 48, 49, 97, 130]))
        special = [0, 1, 4095, 4096, 4097, 8191, 8192, 8193, 16384, 32768, 32769]
        sizes = [int(r.choice(special)) if r.random() < 0.3 else int(r.integers(1, 20000)) for _ in range(nt)]
        cases.append((i, str(r.choice(["sgd", "adagrad", "novograd", "lamb"])), int(r.integers(0, 3)), sizes,
                      bool(r.integers(0, 2)), int(r.integers(0, 1 << 30))))
    return cases


# OSLO_FUZZ_SEED / OSLO_FUZZ_COUNT draw other and longer sweeps, as in test_gpu_random_shapes.py
@pytest.mark.parametrize("i,op,dt,sizes,views,seed",
                         _random_cases(int(os.environ.get("OSLO_FUZZ_COUNT", "48")),
                                       2024 + int(os.environ.get("OSLO_FUZZ_SEED", "0"))))
def test_random_tensor_lists(device, i, op, dt, sizes, views, seed):
    dtype = (F32, F16, BF16)[dt]
    nlists = {"sgd": 3, "adagrad": 3, "novograd": 3, "lamb": 4}[op]
    g = torch.Generator().manual_seed(seed)
    host, devl = [], []
    for k in range(nlists):
        positive = (op == "adagrad" and k == 2) or (op == "lamb" and k == 3)
        if views:
            # every tensor is a view into one buffer, at an offset that is odd for most of them
            offs = np.cumsum([3] + [n + 1 + (j % 3) for j, n in enumerate(sizes)])
            buf = torch.randn(int(offs[-1]) + 8, generator=g)
            buf = (buf.abs() * 0.1 if positive else buf).to(dtype)
            dbuf = buf.to(device)
            host.append([buf[o:o + n] for o, n in zip(offs[:-1], sizes)])
            devl.append([dbuf[o:o + n] for o, n in zip(offs[:-1], sizes)])
        else:
            lst = [torch.randn(n, generator=g) for n in sizes]
            lst = [(t.abs() * 0.1 if positive else t).to(dtype) for t in lst]
            host.append(lst)
            devl.append([t.to(device) for t in lst])
    r = np.random.default_rng(seed)
    lr, wd = float(r.choice([0.01, 0.1])), float(r.choice([0.0, 0.01]))
    picks = sorted(set([0, len(sizes) - 1] + [int(j) for j in r.integers(0, len(sizes), size=6)]))
    out = unrounded(dtype)
    k16 = dict(kw(dtype), min_exact=0.95) if dtype != F32 else {}
    if op == "sgd":
        mu, nest, first = float(r.choice([0.0, 0.9])), bool(r.integers(0, 2)), bool(r.integers(0, 2))
        nest = nest and mu > 0
        _C.get_sgd_kernel().multi_tensor_sgd(0, None, devl, wd, mu, 0.0, lr, nest, first, False, 1.0)
        for j in picks:
            w, m, _ = cf.sgd_step(f64(host[0][j]), f64(host[1][j]), f64(host[2][j]), lr, wd, mu, 0.0, nest, first, out=out)
            if sizes[j]:
                check(devl[1][j], w, "sgd w %d" % j, atol=1e-6, **k16)
                if mu:
                    check(devl[2][j], m, "sgd mom %d" % j, atol=1e-6, **k16)
    elif op == "adagrad":
        mode = int(r.integers(0, 2))
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, None, devl, lr, 1e-10, mode, wd)
        for j in picks:
            p, h = cf.adagrad_step(f64(host[0][j]), f64(host[1][j]), f64(host[2][j]), lr, 1e-10, mode, wd, out=out)
            if sizes[j]:
                check(devl[1][j], p, "adagrad p %d" % j, atol=1e-6, **k16)
                check(devl[2][j], h, "adagrad h %d" % j, atol=1e-7, **k16)
    elif op == "novograd":
        mode, ntype, step = int(r.integers(0, 2)), int(r.choice([0, 2])), int(r.integers(1, 9))
        old = torch.rand(len(sizes), generator=g) + 0.5
        norms = old.to(device)
        _C.get_novograd_kernel().multi_tensor_novograd(0, None, devl, norms, lr, 0.95, 0.98, 1e-8, step, 1, wd, 1,
                                                       mode, ntype)
        got = f64(norms)
        for j in picks:
            n = cf.blend_norm(old[j].item(), f64(host[0][j]), 0.98, 1.0 - 0.98, ntype)
            assert np.isclose(got[j], n, rtol=3e-6), "novograd norm %d" % j
            p, m = cf.novograd_step(f64(host[0][j]), f64(host[1][j]), f64(host[2][j]), got[j], lr, 0.95, 0.98, 1e-8,
                                    step, True, wd, True, mode, out=out)
            if sizes[j]:
                check(devl[1][j], p, "novograd p %d" % j, atol=1e-6, **k16)
                check(devl[2][j], m, "novograd m %d" % j, atol=1e-6, **k16)
    else:
        mode, nv, step = int(r.integers(0, 2)), bool(r.integers(0, 2)), int(r.integers(1, 9))
        clip = float(r.choice([1.0, 1e9]))
        gn = np.float32(np.sqrt(sum(cf.tensor_norm(f64(t)) ** 2 for t in host[0])))
        gnorm = torch.tensor([gn], dtype=torch.float32, device=device)
        _C.get_lamb_kernel().multi_tensor_lamb(0, None, devl, lr, 0.9, 0.999, 1e-6, step, 1, wd, 1, mode, gnorm, clip, nv)
        for j in picks:
            if not sizes[j]:
                continue
            u, m, v = cf.lamb_stage1(f64(host[0][j]), f64(host[1][j]), f64(host[2][j]), f64(host[3][j]), 0.9, 0.999,
                                     1e-6, step, True, wd, True, mode, gn, clip, out=out)
            check(devl[0][j], u, "lamb update %d" % j, atol=1e-6, **k16)
            check(devl[2][j], m, "lamb m %d" % j, atol=1e-7, **k16)
            check(devl[3][j], v, "lamb v %d" % j, atol=1e-8, **k16)
            ud = f64(devl[0][j])
            p = cf.lamb_stage2(ud, f64(host[1][j]), np.float32(cf.tensor_norm(f64(host[1][j]))),
                               np.float32(cf.tensor_norm(ud)), lr, wd, nv, out=out)
            check(devl[1][j], p, "lamb p %d" % j, atol=2e-6, **k16)
    if views:
        # the gaps between the views are untouched
        for k in range(1, nlists):
            full_h = host[k][0]._base if host[k][0]._base is not None else None
            full_d = devl[k][0]._base
            if full_h is None or full_d is None:
                continue
            offs = np.cumsum([3] + [n + 1 + (j % 3) for j, n in enumerate(sizes)])
            gaps = torch.tensor([int(o) - 1 for o in offs])
            assert torch.equal(full_d[gaps.to(device)].cpu(), full_h[gaps]), "gap after list %d" % k
