"""Scaled causal / padding-masked softmax forward and backward on the GPU,
through the C ABI, against the float64 oracle and the reference's unfused torch
chain on identical seeded inputs.  Masked probabilities must be exact zeros."""
import numpy as np
import pytest
import torch

from helpers import check, f64, randn
from oracle import closed_form as cf
from oracle import torch_path as tp
from oslo_amd.torch import _C

pytestmark = pytest.mark.gpu

F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16

CAUSAL_CASES = [
    # (attn_batches, sq, sk, dtype, scale)
    (6, 512, 512, F32, 0.125),      # config-1 row shape
    (3, 128, 128, F32, 0.125),
    (5, 64, 64, BF16, 0.3),
    (2, 2048, 2048, BF16, 0.10206207),  # config-5 row shape
    (2, 1024, 1024, F16, 0.125),
    (3, 37, 64, F16, 0.5),          # sq != sk (sub-sequence of queries)
    (3, 64, 40, BF16, 0.5),         # sq > sk: the first queries see no key
    (1, 8, 4096, BF16, 1.0),        # 8 chunks per lane
    (1, 4, 16384, F16, 1.0),        # several waves per row
    (2, 33, 33, F32, 0.7),          # odd length: scalar kernel
    (2, 9, 100000, BF16, 1.0),      # beyond the register path
    (1, 1, 8, F32, 2.0),
    # lengths that are no multiple of the vector width: one wavefront per row
    # up to 2048 keys, one workgroup per row beyond
    (3, 50, 50, BF16, 0.5),
    (2, 197, 197, F16, 0.125),
    (2, 40, 1001, BF16, 0.25),
    (2, 7, 1027, F16, 0.25),
    (2, 5, 2049, BF16, 0.25),
    (2, 6, 2044, F16, 0.25),
    (5, 3, 1, BF16, 1.0),
    (2, 36, 36, F16, 0.5),          # 8-byte accesses (length a multiple of 4)
    (2, 20, 1004, BF16, 0.25),
    (2, 30, 50, F32, 0.5),          # fp32: 8-byte accesses for even lengths
    (2, 10, 998, F16, 0.25),        # 4-byte accesses
    # rows of exactly 3 x 8 / 16 / 32 / 64 chunks: three chunks per lane
    (3, 192, 192, BF16, 0.25),
    (2, 384, 384, F16, 0.125),
    (2, 768, 768, BF16, 0.125),
    (1, 200, 1536, F16, 0.25),
    (2, 96, 96, F32, 0.5),
    (2, 50, 384, F32, 0.25),
]


@pytest.mark.parametrize("ab,sq,sk,dtype,scale", CAUSAL_CASES)
def test_causal(device, ab, sq, sk, dtype, scale):
    x = randn((ab, sq, sk), dtype, seed=sq + sk)
    dy = randn((ab, sq, sk), dtype, seed=sq + sk + 1)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x.to(device), scale)
    oy = cf.softmax_causal_fwd(f64(x), scale)
    check(y, oy, "causal fwd", atol=1e-9)
    hidden = torch.from_numpy(cf.causal_hidden(sq, sk))
    has_visible = (~hidden).any(-1)
    ycpu = y.cpu()
    assert (ycpu[:, hidden & has_visible[:, None]] == 0).all(), "hidden keys must be exactly 0"
    # backward from the kernel's own output (what autograd saves)
    dx = k.fused_scaled_upper_triang_masked_softmax_backward(dy.to(device), y, scale)
    odx = cf.softmax_bwd(f64(dy), f64(y), scale)
    check(dx, odx, "causal bwd", atol=1e-7)
    assert (dx.cpu()[:, hidden & has_visible[:, None]] == 0).all()
    # in-place variant writes the same values over dy
    g = dy.to(device).clone()
    out = k.fused_scaled_upper_triang_masked_softmax_backward(g, y, scale, inplace=True)
    assert out.data_ptr() == g.data_ptr() and torch.equal(out, dx)


def test_causal_fp32_matches_reference_chain(device):
    """Config-1 semantics: fp32, scale 0.125, -1e4 fill (modeling_gpt2.py:116-138)."""
    x = randn((2, 3, 256, 256), F32, seed=1)
    g = randn((2, 3, 256, 256), F32, seed=2)
    xr = x.clone().requires_grad_()
    ref = tp.causal_softmax(xr, 0.125)
    ref.backward(g)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_upper_triang_masked_softmax_forward(x.view(6, 256, 256).to(device), 0.125)
    dx = k.fused_scaled_upper_triang_masked_softmax_backward(g.view(6, 256, 256).to(device), y, 0.125)
    check(y.view_as(x), f64(ref), "causal fwd vs torch chain", atol=1e-9)
    check(dx.view_as(x), f64(xr.grad), "causal bwd vs torch chain", atol=1e-7)


MASKED_CASES = [
    # (b, np, sq, sk, dtype, scale, mask kind)
    (3, 2, 64, 1024, F16, 0.125, "padding"),    # config-3 row shape, [b,1,1,sk] mask
    (2, 2, 128, 128, BF16, 0.125, "padding"),
    (2, 3, 16, 512, F32, 0.125, "padding"),
    (2, 2, 32, 256, F16, 0.25, "full"),          # [b,1,sq,sk] arbitrary mask
    (2, 2, 32, 256, BF16, 0.25, "shared"),       # [1,1,sq,sk]
    (1, 2, 8, 4096, BF16, 1.0, "padding"),
    (1, 1, 4, 16384, F16, 1.0, "padding"),
    (2, 1, 5, 37, F32, 0.5, "full"),             # scalar kernel
    (2, 2, 16, 64, F16, 1.0, "rows_fully_masked"),
    (2, 2, 16, 64, BF16, 1.0, "none_masked"),
    # scalar kernels with 8-, 4- and 2-byte accesses (mask bytes read 4, 2, 1 at a time)
    (2, 2, 9, 100, F16, 0.5, "full"),
    (2, 2, 9, 50, BF16, 0.5, "padding"),
    (2, 2, 9, 50, BF16, 0.5, "rows_fully_masked"),
    (2, 1, 6, 203, F16, 0.5, "full"),
    (2, 1, 6, 1030, BF16, 0.5, "padding"),
    (2, 1, 6, 2050, BF16, 0.5, "padding"),   # one workgroup per row
    (2, 2, 16, 384, F16, 0.125, "padding"),  # three chunks per lane
    (2, 2, 16, 768, BF16, 0.125, "full"),
    (2, 2, 9, 192, F32, 0.25, "rows_fully_masked"),
]


def make_mask(kind, b, sq, sk, seed):
    r = np.random.default_rng(seed)
    if kind == "padding":
        valid = r.integers(max(1, sk // 4), sk + 1, size=b)
        valid[0] = sk
        return torch.from_numpy(np.arange(sk)[None, :] >= valid[:, None]).view(b, 1, 1, sk)
    if kind == "full":
        m = r.random((b, 1, sq, sk)) < 0.4
        m[..., 0] = False
        return torch.from_numpy(m)
    if kind == "shared":
        m = r.random((1, 1, sq, sk)) < 0.4
        m[..., 0] = False
        return torch.from_numpy(m)
    if kind == "rows_fully_masked":
        m = r.random((b, 1, sq, sk)) < 0.3
        m[:, :, ::3, :] = True
        return torch.from_numpy(m)
    return torch.zeros(b, 1, 1, sk, dtype=torch.bool)


@pytest.mark.parametrize("b,np_,sq,sk,dtype,scale,kind", MASKED_CASES)
def test_masked(device, b, np_, sq, sk, dtype, scale, kind):
    x = randn((b, np_, sq, sk), dtype, seed=sk + sq, std=2.0)
    dy = randn((b, np_, sq, sk), dtype, seed=sk + sq + 1)
    mask = make_mask(kind, b, sq, sk, seed=sk)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), scale)
    oy = cf.softmax_masked_fwd(f64(x), mask.numpy(), scale)
    check(y, oy, "masked fwd", atol=1e-9)
    full = mask.expand(b, np_, sq, sk)
    row_has_visible = (~full).any(-1, keepdim=True).expand_as(full)
    assert (y.cpu()[full & row_has_visible] == 0).all()
    odx = cf.softmax_bwd(f64(dy), f64(y), scale)
    # with the mask (masked loads skipped) and without it (dense read): same result
    dx_m = k.fused_scaled_masked_softmax_backward(dy.to(device), y, scale, mask=mask.to(device))
    dx_d = k.fused_scaled_masked_softmax_backward(dy.to(device), y, scale)
    check(dx_m, odx, "masked bwd (mask given)", atol=1e-7)
    check(dx_d, odx, "masked bwd (dense)", atol=1e-7)
    assert torch.equal(dx_m, dx_d)
    # dx may alias dy: the gradient is overwritten in place, with and without the mask
    g1, g2 = dy.to(device).clone(), dy.to(device).clone()
    r1 = k.fused_scaled_masked_softmax_backward(g1, y, scale, mask=mask.to(device), inplace=True)
    r2 = k.fused_scaled_masked_softmax_backward(g2, y, scale, inplace=True)
    assert r1.data_ptr() == g1.data_ptr() and r2.data_ptr() == g2.data_ptr()
    assert torch.equal(r1, dx_m) and torch.equal(r2, dx_m)


def test_padding_fp16_matches_reference_chain(device):
    """Config-3 semantics against the unfused fp16 chain of the reference
    (modeling_bert.py:298-306).  The chain rounds scale * x and the sum with the
    mask to fp16 before the softmax; scale = 0.125 is exact, so the two paths
    agree to the final rounding."""
    b, h, sq, sk = 2, 2, 64, 512
    x = randn((b, h, sq, sk), F16, seed=5, std=2.0)
    valid = torch.tensor([512, 300])
    pad = torch.arange(sk)[None, :] >= valid[:, None]
    ref = tp.padding_softmax(x, pad, 0.125)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x.to(device), pad.view(b, 1, 1, sk).to(device), 0.125)
    assert (y.cpu() == ref).double().mean() > 0.999
    assert (y.cpu().float() - ref.float()).abs().max() <= 2.0 ** -10


def test_mask_dtypes_and_argument_checks(device):
    k = _C.get_softmax_kernel()
    x = randn((2, 2, 8, 64), F16, 1).to(device)
    m_bool = torch.zeros(2, 1, 1, 64, dtype=torch.bool, device=device)
    m_bool[1, ..., 40:] = True
    a = k.fused_scaled_masked_softmax_forward(x, m_bool, 1.0)
    b = k.fused_scaled_masked_softmax_forward(x, m_bool.to(torch.uint8), 1.0)
    c = k.fused_scaled_masked_softmax_forward(x, m_bool.to(torch.float16), 1.0)
    assert torch.equal(a, b) and torch.equal(a, c)
    with pytest.raises(RuntimeError, match="4D"):
        k.fused_scaled_masked_softmax_forward(x[0], m_bool, 1.0)
    with pytest.raises(RuntimeError, match="3D"):
        k.fused_scaled_upper_triang_masked_softmax_forward(x, 1.0)
    with pytest.raises(RuntimeError, match="broadcast"):
        k.fused_scaled_masked_softmax_forward(x, m_bool[:, :, :, :32], 1.0)
    assert k.get_batch_per_block(1024, 1024, 16, 16) >= 1


def test_row_without_a_visible_key_follows_the_masked_fill_form(device):
    """The two mask forms of the reference differ for a row whose keys are all
    masked: masked_fill(mask, -10000) followed by softmax gives the uniform
    1/sk, the additive form scores * scale + mask
    (oslo/transformers/models/bert/modeling_bert.py:298-306) gives
    softmax(scale * x) because the constant cancels.  The kernel follows the
    masked_fill form; rows that see at least one key are the same in both."""
    b, np_, sq, sk = 2, 2, 8, 64
    x = randn((b, np_, sq, sk), F32, seed=4, std=2.0)
    mask = torch.zeros(b, 1, sq, sk, dtype=torch.bool)
    mask[0, 0, 2, :] = True            # one row without a visible key
    mask[1, 0, :, 40:] = True          # ordinary key padding elsewhere
    scale = 0.25
    filled = torch.softmax((x * scale).masked_fill(mask, -10000.0), dim=-1)
    additive = torch.softmax(x * scale + mask.to(F32) * -10000.0, dim=-1)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), scale).cpu()
    assert torch.allclose(y, filled, rtol=1e-5, atol=1e-7)
    assert torch.equal(y[0, :, 2, :], torch.full((np_, sk), 1.0 / sk))
    # the additive form agrees on every other row and differs on that one
    others = torch.ones(b, np_, sq, dtype=torch.bool)
    others[0, :, 2] = False
    assert torch.allclose(y[others], additive[others], rtol=1e-5, atol=1e-7)
    # (the sum with -10000 is rounded to fp32: the constant cancels up to 1e-3)
    assert torch.allclose(additive[0, :, 2, :], torch.softmax(x[0, :, 2, :] * scale, dim=-1), rtol=5e-3, atol=1e-6)
    assert not torch.allclose(y[0, :, 2, :], additive[0, :, 2, :], rtol=1e-2, atol=1e-4)


@pytest.mark.parametrize("b,np_,sq,sk,dtype", [
    (37, 5, 13, 64, BF16),      # nothing a power of two: batch, heads and queries are recovered by division
    (11, 7, 33, 128, F16),
    (64, 3, 1, 256, BF16),      # one query per head
    (9, 1, 47, 512, F32),       # one head
    (3, 96, 31, 40, BF16),
    (250, 2, 3, 24, F16),
])
def test_row_to_batch_head_query_mapping(device, b, np_, sq, sk, dtype):
    """A kernel row r stands for (batch, head, query) = (r / (np sq), (r / sq) % np,
    r % sq).  Per-batch masks with a different valid length in every batch, and
    the diagonal in causal mode, make any slip in that mapping visible: the
    zeros of a row would sit in the wrong places."""
    x = randn((b, np_, sq, sk), dtype, seed=b + sq, std=2.0)
    r = np.random.default_rng(b * 131 + sk)
    valid = r.integers(1, sk + 1, size=b)
    mask = torch.from_numpy(np.arange(sk)[None, :] >= valid[:, None]).view(b, 1, 1, sk)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), 0.25)
    hidden = np.broadcast_to(mask.numpy(), (b, np_, sq, sk))
    check(y, cf.softmax_masked_fwd(f64(x), hidden, 0.25), "masked fwd", atol=1e-9)
    yc = y.cpu()
    for bi in range(b):
        assert yc[bi, :, :, valid[bi]:].count_nonzero().item() == 0
        assert (yc[bi, :, :, :valid[bi]] > 0).all()
    # per-query masks: the query index matters as well
    pq = torch.from_numpy(r.random((b, 1, sq, sk)) < 0.4)
    pq[..., 0] = False
    y2 = k.fused_scaled_masked_softmax_forward(x.to(device), pq.to(device), 0.25)
    check(y2, cf.softmax_masked_fwd(f64(x), np.broadcast_to(pq.numpy(), (b, np_, sq, sk)), 0.25),
          "per-query mask fwd", atol=1e-9)
    assert (y2.cpu()[pq.expand(b, np_, sq, sk)] == 0).all()
    # causal on [b * np, sq, sk]: the query index of every row
    x3 = x.view(b * np_, sq, sk)
    yc3 = k.fused_scaled_upper_triang_masked_softmax_forward(x3.to(device), 0.25)
    hid = cf.causal_hidden(sq, sk)[None]
    check(yc3, cf.softmax_masked_fwd(f64(x3), np.broadcast_to(hid, (b * np_, sq, sk)), 0.25), "causal fwd", atol=1e-9)
    dy = randn((b * np_, sq, sk), dtype, seed=7)
    dx = k.fused_scaled_upper_triang_masked_softmax_backward(dy.to(device), yc3, 0.25)
    check(dx, cf.softmax_bwd(f64(dy), f64(yc3), 0.25), "causal bwd", atol=1e-7)
    # both at once
    ycm = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), 0.25, causal=True)
    check(ycm, cf.softmax_masked_fwd(f64(x), hidden | hid[None], 0.25), "causal + padding fwd", atol=1e-9)
