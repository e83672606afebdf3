"""Multi-tensor Adam / AdamW on the GPU through the C ABI against the float64
oracle, and FusedAdam against torch.optim on a small model."""
import pytest
import torch

from helpers import NP_NAME, check, f64, randn
from oracle import closed_form as cf
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

SIZES = [1, 7, 2048, 2049, 4096, 8191, 100003, 3, 1 << 20, 0, 12345]


def make_lists(dtype, seed, device):
    gs, ps, ms, vs = [], [], [], []
    for i, n in enumerate(SIZES):
        gs.append(randn((n,), dtype, seed + 4 * i))
        ps.append(randn((n,), dtype, seed + 4 * i + 1))
        ms.append(randn((n,), dtype, seed + 4 * i + 2, std=0.1))
        vs.append(randn((n,), dtype, seed + 4 * i + 3, std=0.1).abs())
    dev = lambda lst: [t.to(device) for t in lst]
    return (gs, ps, ms, vs), (dev(gs), dev(ps), dev(ms), dev(vs))


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("mode,bias_correction,wd", [(1, 1, 0.01), (0, 1, 0.01), (1, 0, 0.0)])
def test_multi_tensor_adam_vs_oracle(device, dtype, mode, bias_correction, wd):
    host, devl = make_lists(dtype, 10, device)
    k = _C.get_adam_kernel()
    lr, b1, b2, eps = 1e-2, 0.9, 0.999, 1e-8
    name = NP_NAME[dtype]
    want = [list(map(f64, lst)) for lst in host]
    for step in (1, 2, 7):
        k.multi_tensor_adam(2048 * 32, None, devl, lr, b1, b2, eps, step, mode, bias_correction, wd)
        for i in range(len(SIZES)):
            p, m, v = cf.adam_step(want[0][i], want[1][i], want[2][i], want[3][i], lr, b1, b2, eps,
                                   step, mode, bias_correction, wd)
            if SIZES[i]:
                # 16-bit: the fp32 evaluation (three roundings before the store) lands
                # on the other side of a tie slightly more often than 0.2 % of the time
                kw = {} if dtype == F32 else {"min_exact": 0.99}
                check(devl[1][i], p, "p[%d] step %d" % (i, step), atol=5e-7, **kw)
                check(devl[2][i], m, "m[%d] step %d" % (i, step), atol=1e-7, **kw)
                check(devl[3][i], v, "v[%d] step %d" % (i, step), atol=1e-8, **kw)
            # continue from what the kernel stored (the stored values are the state)
            want[1][i], want[2][i], want[3][i] = f64(devl[1][i]), f64(devl[2][i]), f64(devl[3][i])
        for i in range(len(SIZES)):
            assert torch.equal(devl[0][i].cpu(), host[0][i]), "gradients must not change"


def test_unaligned_views_and_many_tensors(device):
    """Tensors that start at odd offsets of one buffer (scalar path) and more
    tensors than one launch carries."""
    k = _C.get_adam_kernel()
    n_t, n = 150, 777
    base = [torch.zeros(n_t * (n + 1) + 8, device=device) for _ in range(4)]
    g = torch.Generator(device=device).manual_seed(0)
    for b in base:
        b.normal_(generator=g)
    base[3].abs_()
    ref = [b.clone() for b in base]
    views = [[b[1 + i * (n + 1): 1 + i * (n + 1) + n] for i in range(n_t)] for b in base]
    assert any(v.data_ptr() % 16 for v in views[0])
    k.multi_tensor_adam(0, None, views, 1e-3, 0.9, 0.999, 1e-8, 4, 1, 1, 0.1)
    for i in (0, 1, 63, 64, 65, 149):
        sl = slice(1 + i * (n + 1), 1 + i * (n + 1) + n)
        p, m, v = cf.adam_step(f64(ref[0][sl]), f64(ref[1][sl]), f64(ref[2][sl]), f64(ref[3][sl]),
                               1e-3, 0.9, 0.999, 1e-8, 4, 1, 1, 0.1)
        check(base[1][sl], p, "p view %d" % i, atol=5e-7)
        check(base[2][sl], m, "m view %d" % i, atol=1e-7)
        check(base[3][sl], v, "v view %d" % i, atol=1e-8)
    # the gaps between the views are untouched
    gap = torch.arange(0, n_t * (n + 1) + 8, n + 1, device=device)
    for b, r in zip(base[1:], ref[1:]):
        assert torch.equal(b[gap], r[gap])


def test_argument_checks(device):
    k = _C.get_adam_kernel()
    a = torch.zeros(8, device=device)
    with pytest.raises(RuntimeError):
        k.multi_tensor_adam(0, None, [[a], [a], [a]], 1e-3, 0.9, 0.999, 1e-8, 1, 1, 1, 0.0)
    with pytest.raises(RuntimeError):
        k.multi_tensor_adam(0, None, [[a], [a, a], [a], [a]], 1e-3, 0.9, 0.999, 1e-8, 1, 1, 1, 0.0)
    with pytest.raises(RuntimeError):
        k.multi_tensor_adam(0, None, [[a], [a.half()], [a], [a]], 1e-3, 0.9, 0.999, 1e-8, 1, 1, 1, 0.0)
    with pytest.raises(RuntimeError):
        k.multi_tensor_adam(0, None, [[a], [a], [a], [a]], 1e-3, 0.9, 0.999, 1e-8, 1, 2, 1, 0.0)
    k.multi_tensor_adam(0, None, [[], [], [], []], 1e-3, 0.9, 0.999, 1e-8, 1, 1, 1, 0.0)


@pytest.mark.parametrize("adam_w_mode", [True, False])
def test_fused_adam_optimizer_tracks_torch_optim(device, adam_w_mode):
    """FusedAdam on a small MLP against torch.optim.AdamW / Adam from the same
    start, same gradients, ten steps."""
    from oslo_amd.torch.optim import FusedAdam

    def model():
        torch.manual_seed(0)
        return torch.nn.Sequential(
            torch.nn.Linear(64, 96), torch.nn.GELU(), torch.nn.Linear(96, 33), torch.nn.LayerNorm(33)
        ).to(device)

    a, b = model(), model()
    ref_cls = torch.optim.AdamW if adam_w_mode else torch.optim.Adam
    oa = FusedAdam(a.parameters(), lr=3e-3, weight_decay=0.02, adam_w_mode=adam_w_mode)
    ob = ref_cls(b.parameters(), lr=3e-3, weight_decay=0.02)
    g = torch.Generator(device=device).manual_seed(1)
    for _ in range(10):
        x = torch.randn(16, 64, generator=g, device=device)
        for mdl, opt in ((a, oa), (b, ob)):
            opt.zero_grad()
            mdl(x).square().mean().backward()
            opt.step()
    for pa, pb in zip(a.parameters(), b.parameters()):
        # Adam's normalised update turns a last-bit difference of a tiny gradient
        # into a difference of up to a few 1e-3 * lr in the weight
        assert torch.allclose(pa, pb, rtol=2e-4, atol=5e-5)
    assert oa.param_groups[0]["step"] == 10
    with pytest.raises(RuntimeError):
        FusedAdam(a.parameters(), amsgrad=True)
    with pytest.raises(RuntimeError):
        oa.step(grads=[1])
    oa.zero_grad()
    assert all(p.grad is None for p in a.parameters())


def test_fused_adam_step_details(device):
    """What `step` does around the launch (fused_adam.py:86-184 of the
    reference): a closure is evaluated with gradients enabled and its loss
    returned, parameters without a gradient are left alone, a group without any
    gradient costs nothing, and what the kernel cannot take is refused."""
    from oslo_amd.torch.optim import FusedAdam

    w = torch.nn.Parameter(randn((33,), F32, 1).to(device))
    idle = torch.nn.Parameter(randn((5,), F32, 2).to(device))
    opt = FusedAdam([{"params": [w, idle]}, {"params": [torch.nn.Parameter(torch.zeros(3, device=device))]}],
                    lr=0.1, set_grad_none=False)

    def closure():
        assert torch.is_grad_enabled()
        opt.zero_grad()
        loss = (w * w).sum()
        loss.backward()
        return loss

    before, idle_before = w.detach().clone(), idle.detach().clone()
    with torch.no_grad():
        loss = opt.step(closure)
    assert loss.item() == pytest.approx(float((before * before).sum()))
    assert not torch.equal(w.detach(), before) and torch.equal(idle.detach(), idle_before)
    opt.zero_grad()                      # set_grad_none=False: gradients are zeroed, not dropped
    assert w.grad is not None and not w.grad.any()
    opt.zero_grad(set_to_none=True)
    assert w.grad is None
    with pytest.raises(RuntimeError, match="AMSGrad"):
        FusedAdam([w], amsgrad=True)
    for bad, what in ((torch.nn.Parameter(torch.zeros(4)), "GPU-only"),
                      (torch.nn.Parameter(torch.zeros(4, dtype=torch.float64, device=device)), "fp16, bf16 and fp32"),
                      (torch.nn.Parameter(torch.zeros(4, 6, device=device).t()), "contiguous")):
        o = FusedAdam([bad])
        bad.grad = torch.zeros_like(bad)
        with pytest.raises(RuntimeError, match=what):
            o.step()
    sparse = torch.nn.Parameter(torch.zeros(4, 3, device=device))
    sparse.grad = torch.zeros(4, 3, device=device).to_sparse()
    with pytest.raises(RuntimeError, match="sparse"):
        FusedAdam([sparse]).step()
