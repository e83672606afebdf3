"""What the bindings refuse: the argument checks that the reference's shims
make before a launch (CHECK_INPUT and the shape checks of
oslo/torch/_C/csrc/FusedLayerNormBinder.cpp:8-14, 19-93; the dimension and
dtype checks of FusedScaleMaskSoftmaxBinder.cpp:41-45, 83-86; the list checks
of multi_tensor_apply.cuh:45-70), each raised as RuntimeError before anything
is launched."""
import pytest
import torch

from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16


def _t(device, *shape, dtype=BF16):
    return torch.zeros(*shape, dtype=dtype, device=device)


def test_norm_bindings(device):
    ln = _C.get_layernorm_kernel()
    x, g, b = _t(device, 6, 64), _t(device, 64), _t(device, 64)
    with pytest.raises(RuntimeError, match="at least 1-dimensional"):
        ln.layer_norm_forward(x, (), 1e-5)
    with pytest.raises(RuntimeError, match="expected input with shape"):
        ln.layer_norm_forward(x, (2, 64), 1e-5)
    with pytest.raises(RuntimeError, match="does not match normalized_shape"):
        ln.layer_norm_forward_affine(x, (64,), _t(device, 32), b, 1e-5)
    _, mean, invvar = ln.layer_norm_forward_affine(x, (64,), g, b, 1e-5)
    with pytest.raises(RuntimeError, match="dout of size"):
        ln.layer_norm_backward_affine(_t(device, 5, 64), mean, invvar, x, (64,), g, b, 1e-5)
    with pytest.raises(RuntimeError, match="has dtype"):
        ln.layer_norm_backward_affine(x, mean.to(BF16), invvar, x, (64,), g, b, 1e-5)
    with pytest.raises(RuntimeError, match="elements for"):
        ln.layer_norm_backward_affine(x, mean[:3].contiguous(), invvar, x, (64,), g, b, 1e-5)
    with pytest.raises(RuntimeError, match="gamma has dtype"):
        ln.layer_norm_backward_affine(x, mean, invvar, x, (64,), g.float(), b.float(), 1e-5)
    # the fused residual norm
    _, h, mean, invvar = ln.bias_dropout_add_norm_forward(False, x, b, x, (64,), g, b, 1e-5, 0.1, 1, 0)
    with pytest.raises(RuntimeError, match="dout and h differ"):
        ln.bias_dropout_add_norm_backward(False, x.float(), None, h, mean, invvar, (64,), g, 0.1, 1, 0)
    with pytest.raises(RuntimeError, match="dh_extra and h differ"):
        ln.bias_dropout_add_norm_backward(False, x, _t(device, 5, 64), h, mean, invvar, (64,), g, 0.1, 1, 0)


def test_softmax_bindings(device):
    sm = _C.get_softmax_kernel()
    y4, y3 = _t(device, 2, 2, 4, 64), _t(device, 4, 4, 64)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        sm.fused_scaled_masked_softmax_backward(y3, y3, 1.0)
    with pytest.raises(RuntimeError, match="differ in dtype"):
        sm.fused_scaled_masked_softmax_backward(y4.float(), y4, 1.0)
    with pytest.raises(RuntimeError, match="expected 3D tensor"):
        sm.fused_scaled_upper_triang_masked_softmax_backward(y4, y4, 1.0)
    with pytest.raises(RuntimeError, match="differ in dtype"):
        sm.fused_scaled_upper_triang_masked_softmax_backward(y3.float(), y3, 1.0)
    with pytest.raises(RuntimeError, match="bad shape"):
        sm.get_batch_per_block(0, 64, 2, 2)
    bias = _t(device, 2, 1, 1, 64)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        sm.softmax_bias_backward(y3, y3, 1.0, bias)
    with pytest.raises(RuntimeError, match="differ in dtype"):
        sm.softmax_bias_backward(y4.float(), y4, 1.0, bias)
    with pytest.raises(RuntimeError, match="differ in shape"):
        sm.softmax_bias_backward(_t(device, 2, 2, 3, 64), y4, 1.0, bias)
    stats = torch.zeros(16, 2, dtype=F32, device=device)
    with pytest.raises(RuntimeError, match="differ in dtype or shape"):
        sm.softmax_bias_dropout_backward(y4.float(), y4, bias, stats, 1.0, 0.1, 1, 0)
    with pytest.raises(RuntimeError, match="stats must be float32"):
        sm.softmax_bias_dropout_backward(y4, y4, bias, stats[:5].contiguous(), 1.0, 0.1, 1, 0)
    with pytest.raises(RuntimeError, match="expected 3D tensor"):
        sm.softmax_dropout_backward(y4, y4, stats, None, 1.0, 0.1, 1, 0, causal=True)


def test_elementwise_bindings(device):
    el = _C.get_fused_elementwise_kernel()
    x, b = _t(device, 6, 64), _t(device, 64)
    with pytest.raises(RuntimeError, match="grad_output does not match input"):
        el.bias_gelu_backward(_t(device, 5, 64), x, b)
    with pytest.raises(RuntimeError, match="differ in dtype"):
        el.bias_dropout_add_forward(x, b.float(), None, 0.1, 1, 0)
    with pytest.raises(RuntimeError, match="residual does not match input"):
        el.bias_dropout_add_forward(x, b, _t(device, 5, 64), 0.1, 1, 0)
    assert el.bias_dropout_add_backward(x, 0.1, 1, 0, need_input_grad=False, need_bias_grad=False) == (None, None)
    with pytest.raises(RuntimeError, match="two 64-bit integers"):
        _C.device_rng(torch.zeros(3, dtype=torch.int64, device=device))


def test_multi_tensor_bindings(device):
    g = [_t(device, 10, dtype=F32), _t(device, 7, dtype=F32)]
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    with pytest.raises(RuntimeError, match="Size mismatch"):
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, flag, [g, [_t(device, 10, dtype=F32), _t(device, 8, dtype=F32)], g],
                                                     0.1, 1e-8, 0, 0.0)
    with pytest.raises(RuntimeError, match="must hold"):
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, flag, [g, g], 0.1, 1e-8, 0, 0.0)
    with pytest.raises(RuntimeError, match="int32 tensor on the GPU"):
        _C.get_adagrad_kernel().multi_tensor_adagrad(0, torch.zeros(1, dtype=torch.int32), [g, g, g], 0.1, 1e-8, 0, 0.0)
    k = _C.get_l2norm_kernel()
    with pytest.raises(RuntimeError, match="one list"):
        k.multi_tensor_l2norm(0, flag, [g, g])
    with pytest.raises(RuntimeError, match="no tensors"):
        k.multi_tensor_l2norm(0, flag, [[]])
    k.multi_tensor_norm_out(0, None, [[]], torch.zeros(0, device=device), 0.5, 0.5, 2)   # nothing to do
    sgd = _C.get_sgd_kernel()
    sgd.multi_tensor_sgd(0, flag, [[], [], []], 0.0, 0.9, 0.0, 0.1, False, True, False, 1.0)   # nothing to do
    with pytest.raises(RuntimeError, match="fp16"):
        sgd.multi_tensor_sgd(0, flag, [g, g, g, g], 0.0, 0.9, 0.0, 0.1, False, True, False, 1.0)
    nv = _C.get_novograd_kernel()
    with pytest.raises(RuntimeError, match="must hold"):
        nv.multi_tensor_novograd(0, flag, [g, g], torch.zeros(2, device=device), 0.1, 0.9, 0.99, 1e-8, 1, 1, 0.0, 1,
                                 0, 2)
    lamb = _C.get_lamb_kernel()
    gn = torch.ones(1, device=device)
    with pytest.raises(RuntimeError, match="must hold"):
        lamb.multi_tensor_lamb(0, flag, [g, g, g], 0.1, 0.9, 0.99, 1e-6, 1, 1, 0.0, 1, 1, gn, 1.0, False)
    with pytest.raises(RuntimeError, match="float32"):
        lamb.multi_tensor_lamb(0, flag, [g, g, g, g], 0.1, 0.9, 0.99, 1e-6, 1, 1, 0.0, 1, 1, gn.to(BF16), 1.0, False)
    mp = _C.get_lamb_mp_kernel()
    f = lambda v, dt=F32: torch.tensor([v], dtype=dt, device=device)
    args = (f(0.1), 0.9, 0.99, 1e-6, f(1, torch.int32), 1, 0.0, 1, 1, gn, f(1.0), False, f(0.0), f(1.0))
    with pytest.raises(RuntimeError, match="4 or 5 lists"):
        mp.multi_tensor_lamb_mp(0, flag, [g, g, g], *args)
    h = [t.to(F16) for t in g]
    with pytest.raises(RuntimeError, match="master values"):
        mp.multi_tensor_lamb_mp(0, flag, [h, h, h, h, h], *args)
    with pytest.raises(RuntimeError, match="share one dtype"):
        mp.multi_tensor_lamb_mp(0, flag, [h, g, g, g], *args)
    with pytest.raises(RuntimeError, match="overflow flag"):
        mp.multi_tensor_lamb_mp(0, None, [g, g, g, g], *args)
    with pytest.raises(RuntimeError, match="tensor on"):
        mp.multi_tensor_lamb_mp(0, flag, [g, g, g, g], torch.tensor([0.1]), *args[1:])
