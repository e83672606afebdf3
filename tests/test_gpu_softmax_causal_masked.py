"""Causal mask and padding mask in one softmax call (the attention of a causal
model on a padded batch, oslo/transformers/models/gpt2/modeling_gpt2.py:126-136,
573-581), forward and backward, with and without the fused dropout, on the GPU
through the C ABI.

Oracle: the float64 masked softmax with hidden = causal | padding
(oracle/closed_form.py), whose convention for a row without a visible key is the
uniform 1/sk; the reference's own unfused chain (where + additive mask) is
compared where every row sees a key.  Hidden probabilities are exact zeros and
the dropout keep bits are those of the integer Philox oracle, bit for bit."""
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


def key_mask(kind, b, sk, seed):
    """[b, 1, 1, sk] boolean, True = padded key."""
    r = np.random.default_rng(seed)
    m = np.zeros((b, sk), dtype=bool)
    if kind == "right":          # valid prefix, sample 0 unpadded
        valid = r.integers(max(1, sk // 4), sk + 1, size=b)
        valid[0] = sk
        m = np.arange(sk)[None, :] >= valid[:, None]
    elif kind == "left":         # padded prefix: the first queries see no key at all
        pad = r.integers(1, max(2, sk // 2), size=b)
        pad[0] = 0
        m = np.arange(sk)[None, :] < pad[:, None]
    elif kind == "one_sample_all_padded":
        valid = r.integers(max(1, sk // 4), sk + 1, size=b)
        m = np.arange(sk)[None, :] >= valid[:, None]
        m[-1, :] = True
    elif kind == "holes":
        m = r.random((b, sk)) < 0.3
    return torch.from_numpy(m).view(b, 1, 1, sk)


def hidden_of(mask, b, sq, sk):
    """[b, 1, sq, sk] numpy: padding | beyond the diagonal."""
    return mask.expand(b, 1, sq, sk).numpy() | cf.causal_hidden(sq, sk)[None, None]


CASES = [
    # (b, np, sq, sk, dtype, scale, kind)
    (3, 2, 128, 128, BF16, 0.125, "right"),
    (2, 2, 512, 512, F32, 0.125, "right"),
    (2, 2, 256, 2048, BF16, 0.10206207, "right"),      # config-5 row length, sq != sk
    (2, 3, 64, 1024, F16, 0.125, "holes"),
    (3, 2, 96, 96, BF16, 0.3, "left"),                  # rows without a visible key
    (3, 2, 64, 64, F16, 0.5, "one_sample_all_padded"),
    (2, 2, 37, 64, F16, 0.5, "right"),                  # sq < sk
    (2, 2, 64, 40, BF16, 0.5, "right"),                 # sq > sk: the diagonal hides whole rows
    (1, 2, 8, 4096, BF16, 1.0, "right"),                # two waves per row
    (2, 1, 4, 16384, F16, 1.0, "holes"),
    (2, 2, 33, 33, F32, 0.7, "right"),                  # odd length: scalar kernels
    (2, 2, 50, 50, BF16, 0.5, "left"),
    (2, 2, 20, 1004, BF16, 0.25, "holes"),
    (2, 1, 5, 2051, BF16, 0.25, "right"),               # one workgroup per row
    (2, 2, 192, 192, BF16, 0.25, "right"),              # three chunks per lane
    (2, 2, 100, 768, F16, 0.125, "holes"),
    (3, 1, 1, 8, F32, 2.0, "right"),
    # sq > sk where rows lie side by side in a wave: queries without any key next to queries that see keys
    (2, 2, 73, 64, BF16, 0.25, "right"),
    (2, 2, 137, 128, F16, 0.25, "holes"),
    (2, 2, 41, 32, F32, 0.25, "left"),
    (2, 2, 300, 256, BF16, 0.25, "right"),
]


@pytest.mark.parametrize("b,np_,sq,sk,dtype,scale,kind", CASES)
def test_causal_masked(device, b, np_, sq, sk, dtype, scale, kind):
    x = randn((b, np_, sq, sk), dtype, seed=sq + sk, std=2.0)
    dy = randn((b, np_, sq, sk), dtype, seed=sq + sk + 1)
    mask = key_mask(kind, b, sk, seed=sk)
    hidden = hidden_of(mask, b, sq, sk)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), scale, causal=True)
    oy = cf.softmax_masked_fwd(f64(x), hidden, scale)
    check(y, oy, "causal+padding fwd", atol=1e-9)
    full = torch.from_numpy(np.broadcast_to(hidden, (b, np_, sq, sk)).copy())
    row_has_visible = (~full).any(-1, keepdim=True).expand_as(full)
    assert (y.cpu()[full & row_has_visible] == 0).all(), "hidden keys must be exactly 0"
    # the same answer from the padding-mask kernel fed the combined mask
    y2 = k.fused_scaled_masked_softmax_forward(x.to(device), torch.from_numpy(hidden).to(device), scale)
    assert torch.equal(y, y2)
    odx = cf.softmax_bwd(f64(dy), f64(y), scale)
    dx_m = k.fused_scaled_masked_softmax_backward(dy.to(device), y, scale, mask=mask.to(device), causal=True)
    dx_d = k.fused_scaled_masked_softmax_backward(dy.to(device), y, scale, causal=True)
    check(dx_m, odx, "causal+padding bwd (mask given)", atol=1e-7)
    check(dx_d, odx, "causal+padding bwd (no mask)", atol=1e-7)
    assert torch.equal(dx_m, dx_d)
    gi = dy.to(device).clone()
    ri = k.fused_scaled_masked_softmax_backward(gi, y, scale, mask=mask.to(device), inplace=True, causal=True)
    assert ri.data_ptr() == gi.data_ptr() and torch.equal(ri, dx_m)  # dx may alias dy


def test_matches_the_reference_chain_where_every_row_sees_a_key(device):
    """modeling_gpt2.py:126-136: where(causal, w, -1e4) + attention_mask with
    (1 - m) * -10000, softmax, in fp32."""
    b, np_, sq, sk = 3, 4, 96, 96
    x = randn((b, np_, sq, sk), F32, seed=3, std=2.0)
    mask = key_mask("right", b, sk, seed=1)
    scale = 0.125
    w = x * scale
    causal = torch.tril(torch.ones(sk, sk, dtype=torch.bool))[sk - sq:sk, :sk]
    w = torch.where(causal, w, torch.tensor(-1e4))
    w = w + mask.to(torch.float32) * -10000.0
    ref = torch.softmax(w, dim=-1)
    k = _C.get_softmax_kernel()
    y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), scale, causal=True).cpu()
    assert torch.allclose(y, ref, rtol=1e-5, atol=1e-7)
    assert (y[ref == 0] == 0).all()


def test_per_query_mask_and_shared_mask(device):
    """mask_sq == sq and mask_b == 1 broadcast forms with the diagonal on top."""
    b, np_, sq, sk = 2, 2, 48, 256
    x = randn((b, np_, sq, sk), BF16, seed=11, std=2.0)
    k = _C.get_softmax_kernel()
    for kind in ("full", "shared"):
        mask = make_mask(kind, b, sq, sk, seed=3)
        hidden = mask.expand(b, 1, sq, sk).numpy() | cf.causal_hidden(sq, sk)[None, None]
        y = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), 0.25, causal=True)
        check(y, cf.softmax_masked_fwd(f64(x), hidden, 0.25), "causal + %s mask" % kind, atol=1e-9)


DROPOUT_CASES = [
    (2, 2, 128, 128, BF16, 0.125, "right", 0.1),
    (2, 2, 512, 512, F32, 0.125, "right", 0.1),
    (2, 2, 64, 2048, BF16, 0.10206207, "holes", 0.1),
    (3, 2, 64, 64, F16, 0.5, "one_sample_all_padded", 0.2),
    (3, 2, 96, 96, BF16, 0.3, "left", 0.1),
    (2, 2, 37, 64, F16, 0.5, "right", 0.1),
    (2, 2, 33, 33, F32, 0.7, "right", 0.1),
    (2, 1, 5, 2051, BF16, 0.25, "right", 0.1),
    # sq > sk where rows lie side by side in a wave: queries without any key next to queries that see keys
    (2, 2, 73, 64, BF16, 0.25, "right", 0.1),
    (2, 2, 137, 128, F16, 0.25, "holes", 0.1),
    (2, 2, 41, 32, F32, 0.25, "left", 0.1),
]


@pytest.mark.parametrize("b,np_,sq,sk,dtype,scale,kind,p", DROPOUT_CASES)
def test_causal_masked_dropout(device, b, np_, sq, sk, dtype, scale, kind, p):
    seed, offset = 77 + sk, 4 * sq
    x = randn((b, np_, sq, sk), dtype, seed=sq + sk, std=2.0)
    g = randn((b, np_, sq, sk), dtype, seed=sq + sk + 1)
    mask = key_mask(kind, b, sk, seed=sk)
    hidden = hidden_of(mask, b, sq, sk)
    k = _C.get_softmax_kernel()
    out, stats = k.softmax_dropout_forward(x.to(device), mask.to(device), scale, p, seed, offset, causal=True)
    n = b * np_ * sq * sk
    keep = philox.keep_mask(n, p, seed, offset).reshape(b, np_, sq, sk).astype(bool)
    oo = cf.softmax_dropout_fwd(f64(x), hidden, scale, keep, p)
    check(out, oo, "causal+padding dropout fwd", atol=1e-9)
    # the keep decisions are the Philox stream over the flattened output, bit for bit:
    # a kept, visible probability is non-zero, a dropped one exactly zero
    ocpu = out.cpu()
    assert (ocpu[torch.from_numpy(~keep)] == 0).all(), "dropped elements must be exactly 0"
    plain = k.fused_scaled_masked_softmax_forward(x.to(device), mask.to(device), scale, causal=True).cpu()
    kept_visible = torch.from_numpy(keep) & (plain != 0)
    assert (ocpu[kept_visible] != 0).all(), "kept elements must survive"
    dx = k.softmax_dropout_backward(g.to(device), x.to(device), stats, mask.to(device), scale, p, seed, offset,
                                    causal=True)
    odx = cf.softmax_dropout_bwd(f64(g), f64(x), hidden, scale, keep, p)
    check(dx, odx, "causal+padding dropout bwd", atol=2e-7)
    # p = 0 reproduces the plain kernel bit for bit
    out0, _ = k.softmax_dropout_forward(x.to(device), mask.to(device), scale, 0.0, seed, offset, causal=True)
    assert torch.equal(out0.cpu(), plain)


def test_autograd_and_module(device):
    import oslo_amd.torch.nn as onn
    from oslo_amd.torch.nn.modules.softmax import AttnMaskType, FusedScaleMaskSoftmax

    b, np_, sq, sk = 2, 3, 64, 64
    x = randn((b, np_, sq, sk), F32, seed=2, std=2.0)
    dy = randn((b, np_, sq, sk), F32, seed=3)
    mask = key_mask("right", b, sk, seed=5)
    hidden = torch.from_numpy(hidden_of(mask, b, sq, sk))
    xd = x.to(device).requires_grad_()
    y = onn.scaled_masked_softmax(xd, mask.to(device), 0.25, causal=True)
    y.backward(dy.to(device))
    xr = x.clone().requires_grad_()
    ref = torch.softmax((xr * 0.25).masked_fill(hidden, float("-inf")), dim=-1)
    ref.backward(dy)
    assert torch.allclose(y.cpu(), ref, rtol=1e-5, atol=1e-7)
    assert torch.allclose(xd.grad.cpu(), xr.grad, rtol=1e-5, atol=1e-6)
    # the module with the causal type takes a key-padding mask and applies the diagonal itself;
    # its torch branch (fusion off) gives the same probabilities
    fused = FusedScaleMaskSoftmax(attn_mask_type=AttnMaskType.causal, scale=0.25)
    unfused = FusedScaleMaskSoftmax(attn_mask_type=AttnMaskType.causal, scale=0.25,
                                    scaled_masked_softmax_fusion=False)
    a = fused(x.to(device), mask.to(device)).cpu()
    c = unfused(x.to(device), mask.to(device)).cpu()
    assert torch.allclose(a, ref.detach(), rtol=1e-5, atol=1e-7)
    assert torch.allclose(c, ref.detach(), rtol=1e-5, atol=1e-6)
