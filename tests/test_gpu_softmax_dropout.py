"""Softmax with the attention-probability dropout fused in, forward and
backward on the GPU through the C ABI, against the float64 oracle with the keep
mask of the integer Philox oracle on identical seeded inputs."""
import numpy as np
import pytest
import torch

from helpers import check, f64, randn
from oracle import closed_form as cf
from oracle import philox
from oslo_amd.torch import _C
from test_gpu_softmax import make_mask

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16


def oracle_keep(shape, p, seed, offset):
    n = int(np.prod(shape))
    return philox.keep_mask(n, p, seed, offset).reshape(shape).astype(bool)


CAUSAL_CASES = [
    # (attn_batches, sq, sk, dtype, scale, p)
    (3, 128, 128, F32, 0.125, 0.1),       # 4-element chunks: half a Philox group each
    (2, 512, 512, F32, 0.125, 0.1),       # config-1 row shape
    (5, 64, 64, BF16, 0.3, 0.1),
    (2, 2048, 2048, BF16, 0.10206207, 0.1),  # config-5 row shape
    (2, 1024, 1024, F16, 0.125, 0.5),
    (3, 37, 64, F16, 0.5, 0.1),           # sq != sk
    (3, 64, 40, BF16, 0.5, 0.2),          # sq > sk: queries without a visible key
    (1, 8, 4096, BF16, 1.0, 0.1),
    (1, 4, 16384, F16, 1.0, 0.1),         # several waves per row
    (2, 33, 33, F32, 0.7, 0.1),           # odd length: scalar kernel
    (2, 5, 100000, BF16, 1.0, 0.1),       # beyond the register path
    (1, 1, 8, F32, 2.0, 0.3),
    (2, 16, 64, BF16, 1.0, 1.0),          # p = 1: everything dropped
    (3, 50, 50, BF16, 0.5, 0.1),          # one wavefront per row, scalar accesses
    (2, 197, 197, F16, 0.125, 0.2),
    (2, 9, 1001, BF16, 0.25, 0.1),
    (2, 5, 2046, F16, 0.25, 0.1),
    (2, 5, 2051, BF16, 0.25, 0.1),        # one workgroup per row
    (4, 5, 1, F32, 1.0, 0.3),             # one key: the gradient is exactly zero
    (2, 384, 384, BF16, 0.125, 0.1),      # three chunks per lane
    (2, 100, 768, F16, 0.125, 0.2),
    (2, 60, 192, F32, 0.25, 0.1),
]


@pytest.mark.parametrize("ab,sq,sk,dtype,scale,p", CAUSAL_CASES)
def test_causal_dropout(device, ab, sq, sk, dtype, scale, p):
    seed, offset = 1234 + sk, 8 * sq
    x = randn((ab, sq, sk), dtype, seed=sq + sk)
    g = randn((ab, sq, sk), dtype, seed=sq + sk + 1)
    k = _C.get_softmax_kernel()
    out, stats = k.softmax_dropout_forward(x.to(device), None, scale, p, seed, offset)
    keep = oracle_keep((ab, sq, sk), p, seed, offset)
    hidden = cf.causal_hidden(sq, sk)
    oo = cf.softmax_dropout_fwd(f64(x), hidden, scale, keep, p)
    check(out, oo, "causal dropout fwd", atol=1e-9)
    # exact zeros: every dropped element and every hidden key of a row that sees a key
    ocpu = out.cpu()
    assert (ocpu[torch.from_numpy(~keep)] == 0).all(), "dropped elements must be exactly 0"
    has_visible = (~torch.from_numpy(hidden)).any(-1)
    assert (ocpu[:, torch.from_numpy(hidden) & has_visible[:, None]] == 0).all()
    dx = k.softmax_dropout_backward(g.to(device), x.to(device), stats, None, scale, p, seed, offset)
    odx = cf.softmax_dropout_bwd(f64(g), f64(x), hidden, scale, keep, p)
    check(dx, odx, "causal dropout bwd", atol=2e-7)
    # in place over the gradient
    gi = g.to(device).clone()
    r = k.softmax_dropout_backward(gi, x.to(device), stats, None, scale, p, seed, offset, inplace=True)
    assert r.data_ptr() == gi.data_ptr() and torch.equal(r, dx)


MASKED_CASES = [
    # (b, np, sq, sk, dtype, scale, kind, p)
    (2, 3, 64, 1024, F16, 0.125, "padding", 0.1),    # config-3 row shape
    (2, 2, 32, 256, BF16, 0.125, "full", 0.1),
    (2, 2, 16, 512, F32, 0.25, "shared", 0.2),
    (2, 2, 12, 64, BF16, 1.0, "rows_fully_masked", 0.1),
    (2, 2, 7, 50, F16, 0.5, "full", 0.1),            # scalar kernel
    (1, 2, 4, 8192, BF16, 1.0, "padding", 0.1),
    (3, 1, 9, 128, F32, 0.3, "none", 0.4),
    (2, 2, 12, 100, F16, 0.5, "full", 0.1),          # scalar kernel, 8-byte accesses
    (2, 2, 12, 50, BF16, 0.5, "padding", 0.2),       # 4-byte accesses
    (2, 2, 12, 50, F32, 0.5, "full", 0.1),           # fp32, 8-byte accesses
    (2, 2, 12, 77, BF16, 0.5, "rows_fully_masked", 0.1),
    (2, 2, 12, 768, F16, 0.125, "full", 0.1),        # three chunks per lane
    (2, 2, 12, 1536, BF16, 0.125, "padding", 0.1),
]


@pytest.mark.parametrize("b,np_,sq,sk,dtype,scale,kind,p", MASKED_CASES)
def test_masked_dropout(device, b, np_, sq, sk, dtype, scale, kind, p):
    seed, offset = 99 + sk, 4 * sq
    x = randn((b, np_, sq, sk), dtype, seed=sk + sq, std=2.0)
    g = randn((b, np_, sq, sk), dtype, seed=sk + sq + 1)
    mask = make_mask(kind, b, sq, sk, seed=sk)
    k = _C.get_softmax_kernel()
    out, stats = k.softmax_dropout_forward(x.to(device), mask.to(device), scale, p, seed, offset)
    keep = oracle_keep((b, np_, sq, sk), p, seed, offset)
    oo = cf.softmax_dropout_fwd(f64(x), mask.numpy(), scale, keep, p)
    check(out, oo, "masked dropout fwd", atol=1e-9)
    assert (out.cpu()[torch.from_numpy(~keep)] == 0).all()
    dx = k.softmax_dropout_backward(
        g.to(device), x.to(device), stats, mask.to(device), scale, p, seed, offset
    )
    odx = cf.softmax_dropout_bwd(f64(g), f64(x), mask.numpy(), scale, keep, p)
    check(dx, odx, "masked dropout bwd", atol=2e-7)


@pytest.mark.parametrize("dtype,sk", [(F32, 512), (BF16, 2048), (F16, 1000), (BF16, 77)])
def test_p_zero_equals_plain_softmax_bit_for_bit(device, dtype, sk):
    x = randn((3, 40, sk), dtype, seed=5).to(device)
    k = _C.get_softmax_kernel()
    out, stats = k.softmax_dropout_forward(x, None, 0.2, 0.0, 1, 0)
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x, 0.2)
    assert torch.equal(out, y)
    # statistics: exp2(log2-domain logit - max) * inv reproduces the probabilities
    xs = f64(x) * (0.2 * np.log2(np.e))
    st = f64(stats).reshape(3, 40, 2)
    hidden = cf.causal_hidden(40, sk)
    rec = np.where(hidden, 0.0, np.exp2(xs - st[..., :1]) * st[..., 1:])
    assert np.allclose(rec, cf.softmax_causal_fwd(f64(x), 0.2), rtol=3e-6, atol=1e-12)
    # backward with p = 0 equals the plain backward up to the rounding of the saved y
    g = randn((3, 40, sk), dtype, seed=6).to(device)
    dx = k.softmax_dropout_backward(g, x, stats, None, 0.2, 0.0, 1, 0)
    check(dx, cf.softmax_bwd(f64(g), cf.softmax_causal_fwd(f64(x), 0.2), 0.2), "p=0 bwd", atol=2e-7)


def test_keep_mask_is_the_philox_stream_of_the_elementwise_ops(device):
    """Same (p, seed, offset) => the same keep decisions as oslo_philox_mask over
    the flattened output, for 8- and 4-element chunks and the scalar kernel."""
    ek = _C.get_fused_elementwise_kernel()
    k = _C.get_softmax_kernel()
    for dtype, sk in ((BF16, 256), (F32, 256), (F32, 36), (F16, 30)):
        x = torch.zeros(2, 3, 5, sk, dtype=dtype, device=device)
        mask = torch.zeros(1, 1, 1, sk, dtype=torch.bool, device=device)
        out, _ = k.softmax_dropout_forward(x, mask, 1.0, 0.3, 77, 12)
        m = ek.philox_mask(x.numel(), 0.3, 77, 12, device).view_as(x).bool()
        assert torch.equal(out != 0, m)
        kept = out[m].float()
        assert torch.allclose(kept, torch.full_like(kept, (1.0 / sk) / 0.7), rtol=4e-3)


def test_argument_checks(device):
    k = _C.get_softmax_kernel()
    x = torch.zeros(2, 4, 8, device=device)
    with pytest.raises(RuntimeError):
        k.softmax_dropout_forward(x, None, 1.0, 1.5, 0, 0)
    with pytest.raises(RuntimeError):
        k.softmax_dropout_forward(x.view(2, 2, 2, 8), None, 1.0, 0.1, 0, 0)
    out, stats = k.softmax_dropout_forward(x, None, 1.0, 0.1, 0, 0)
    with pytest.raises(RuntimeError):
        k.softmax_dropout_backward(x, x, stats[:3], None, 1.0, 0.1, 0, 0)
    with pytest.raises(RuntimeError):
        k.softmax_dropout_backward(x.half(), x, stats, None, 1.0, 0.1, 0, 0)


def test_module_and_autograd(device):
    """FusedScaleMaskSoftmax(attn_dropout=p): training mode drops with the
    generator's Philox state and backpropagates to the scores; eval mode and
    p = 0 are the plain softmax."""
    import oslo_amd.torch.nn as onn

    b, np_, s = 2, 3, 128
    x = randn((b, np_, s, s), BF16, seed=3).to(device).requires_grad_(True)
    m = onn.FusedScaleMaskSoftmax(
        input_in_bf16=True, attn_mask_type=onn.AttnMaskType.causal, scale=0.25, attn_dropout=0.1
    ).to(device)
    torch.manual_seed(321)
    gen = torch.cuda.default_generators[x.device.index or 0]
    seed, offset = gen.initial_seed(), gen.get_offset()
    out = m(x, None)
    assert gen.get_offset() == offset + 4
    keep = oracle_keep((b * np_, s, s), 0.1, seed, offset)
    hidden = cf.causal_hidden(s, s)
    oo = cf.softmax_dropout_fwd(f64(x).reshape(b * np_, s, s), hidden, 0.25, keep, 0.1)
    check(out.reshape(b * np_, s, s), oo, "module fwd", atol=1e-9)
    g = randn((b, np_, s, s), BF16, seed=4).to(device)
    out.backward(g)
    odx = cf.softmax_dropout_bwd(
        f64(g).reshape(b * np_, s, s), f64(x).reshape(b * np_, s, s), hidden, 0.25, keep, 0.1
    )
    check(x.grad.reshape(b * np_, s, s), odx, "module bwd", atol=2e-7)
    m.eval()
    plain = onn.FusedScaleMaskSoftmax(
        input_in_bf16=True, attn_mask_type=onn.AttnMaskType.causal, scale=0.25
    )
    assert torch.equal(m(x, None), plain(x, None))
    # padding form through the module
    m.train()
    pm = onn.FusedScaleMaskSoftmax(input_in_bf16=True, scale=0.25, attn_dropout=0.2).to(device)
    mask = make_mask("padding", b, s, s, seed=1).to(device)
    seed, offset = gen.initial_seed(), gen.get_offset()
    o2 = pm(x.detach(), mask)
    keep2 = oracle_keep((b, np_, s, s), 0.2, seed, offset)
    check(o2, cf.softmax_dropout_fwd(f64(x), mask.cpu().numpy(), 0.25, keep2, 0.2), "module padding fwd", atol=1e-9)
