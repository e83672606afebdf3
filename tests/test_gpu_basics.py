"""GPU checks of the shared device building blocks, through the C ABI:
wave64 DPP reductions, Philox4x32-10 words and keep-mask (bit-exact against the
integer oracle), and the copy probe."""
import numpy as np
import pytest
import torch

from oracle import philox
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu


def test_wave_reduce_selftest(device):
    out = _C.get_fused_elementwise_kernel().wave_reduce_selftest(device).cpu().tolist()
    assert out == [2016.0, 63.0, 2016.0, 4032.0]


@pytest.mark.parametrize(
    "seed,offset,first",
    [(0, 0, 0), (1234, 0, 0), (0x0123456789ABCDEF, 0x00000002FFFFFFFF, 2 ** 32 - 3), (2 ** 64 - 1, 2 ** 64 - 4, 7)],
)
def test_philox_words_bit_exact(device, seed, offset, first):
    n = 1000
    got = _C.get_fused_elementwise_kernel().philox_words(n, first, seed, offset, device)
    got = got.cpu().numpy().view(np.uint32).reshape(n, 4)
    want = philox.group_words(first, n, seed, offset)
    assert np.array_equal(got, want)


def test_philox_known_answer_on_device(device):
    # counter (0,0,0,0), key (0,0) -> Random123 vector
    got = _C.get_fused_elementwise_kernel().philox_words(1, 0, 0, 0, device)
    got = got.cpu().numpy().view(np.uint32)
    assert [int(v) for v in got] == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]


@pytest.mark.parametrize("n", [1, 7, 8, 9, 4097, 1 << 20])
@pytest.mark.parametrize("p", [0.0, 0.1, 0.5, 1.0])
def test_philox_mask_bit_exact(device, n, p):
    got = _C.get_fused_elementwise_kernel().philox_mask(n, p, 1234, 8, device).cpu().numpy()
    want = philox.keep_mask(n, p, 1234, 8)
    assert np.array_equal(got, want)


def test_copy_probe(device):
    src = torch.arange(1 << 22, dtype=torch.int32, device=device)
    dst = torch.zeros_like(src)
    _C.get_fused_elementwise_kernel().copy_probe(src, dst)
    assert torch.equal(src, dst)
    small = torch.arange(12, dtype=torch.int32, device=device)
    out = torch.zeros_like(small)
    _C.get_fused_elementwise_kernel().copy_probe(small, out)
    assert torch.equal(small, out)


def test_binding_refuses_operands_that_do_not_fit(device):
    """The kernels read through raw pointers, so the binding has to turn away
    what would make them read outside a buffer: a mask in host memory, gradients
    of another shape, statistics of the wrong length."""
    from oslo_amd.torch._C import get_fused_elementwise_kernel, get_layernorm_kernel, get_softmax_kernel

    sm, ln, el = get_softmax_kernel(), get_layernorm_kernel(), get_fused_elementwise_kernel()
    x = torch.randn(2, 3, 8, 16, device=device)
    y = torch.softmax(x, -1)
    mask = torch.zeros(2, 1, 1, 16, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="mask is on"):
        sm.fused_scaled_masked_softmax_forward(x, mask, 1.0)
    with pytest.raises(RuntimeError, match="mask is on"):
        sm.fused_scaled_masked_softmax_backward(y, y, 1.0, mask=mask)
    with pytest.raises(RuntimeError, match="does not broadcast"):
        sm.fused_scaled_masked_softmax_backward(y, y, 1.0, mask=torch.zeros(2, 1, 1, 8, dtype=torch.bool, device=device))
    with pytest.raises(RuntimeError, match="differ in shape"):
        sm.fused_scaled_masked_softmax_backward(y[:, :, :4].contiguous(), y, 1.0)
    y3 = y.view(6, 8, 16)
    with pytest.raises(RuntimeError, match="differ in shape"):
        sm.fused_scaled_upper_triang_masked_softmax_backward(y3[:3].contiguous(), y3, 1.0)

    h = torch.randn(12, 64, device=device)
    out, mean, invvar = ln.layer_norm_forward(h, (64,), 1e-5)
    with pytest.raises(RuntimeError, match="elements for 12 rows"):
        ln.layer_norm_backward(out, mean[:6].contiguous(), invvar, h, (64,), 1e-5)
    with pytest.raises(RuntimeError, match="one element per row"):
        ln.bias_dropout_add_norm_backward(False, out, None, h, mean, invvar[:6].contiguous(), (64,), None, 0.0, 0, 0)
    with pytest.raises(RuntimeError, match="gamma has dtype"):
        ln.bias_dropout_add_norm_backward(False, out, None, h, mean, invvar, (64,),
                                          torch.ones(64, device=device, dtype=torch.float16), 0.0, 0, 0)
    with pytest.raises(RuntimeError, match="differ in dtype"):
        el.bias_gelu_backward(out, h, torch.zeros(64, device=device, dtype=torch.float16))
