"""Model-level drop-in: a randomly initialised Hugging Face GPT-2 / T5 block
routed through the fused ops by oslo_amd.transformers (the counterpart of the
reference's oslo/transformers/kernel_fusion_utils.py), against the same model on
its unfused eager path.  The CPU cases run the host logic and the torch
fallbacks; the GPU cases run the kernels."""
import pytest
import torch

transformers = pytest.importorskip("transformers")

from oslo_amd.transformers import (  # noqa: E402
    fused_layer_norm,
    fused_rms_norm,
    fused_scale_mask_softmax,
)
import oslo_amd.torch.nn as onn  # noqa: E402


def tiny_gpt2(seed=0, **kw):
    from transformers import GPT2Config, GPT2LMHeadModel

    cfg = GPT2Config(n_layer=2, n_head=4, n_embd=128, vocab_size=211, n_positions=128,
                     bos_token_id=0, eos_token_id=0, **kw)
    torch.manual_seed(seed)
    m = GPT2LMHeadModel(cfg)
    m.config._attn_implementation = "eager"
    return m


def inputs(b=3, s=48, vocab=211, seed=1):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab, (b, s), generator=g)
    am = torch.ones(b, s, dtype=torch.long)
    am[1, s - 11:] = 0
    am[2, s // 2:] = 0
    return ids, am


def test_swaps_on_cpu_keep_the_model_output():
    m = tiny_gpt2().eval()
    ids, am = inputs()
    ref_causal = m(ids).logits
    ref_padded = m(ids, attention_mask=am).logits
    assert fused_layer_norm(m) == 5  # 2 x (ln_1, ln_2) + ln_f
    assert all(type(x) is not torch.nn.LayerNorm for x in m.modules())
    assert sum(isinstance(x, onn.FusedLayerNorm) for x in m.modules()) == 5
    fused_scale_mask_softmax(m)
    assert m.config._attn_implementation == "oslo_fused_softmax"
    out = m(ids).logits
    assert torch.allclose(out, ref_causal, atol=1e-5, rtol=1e-5)
    out = m(ids, attention_mask=am).logits
    valid = am.bool()
    assert torch.allclose(out[valid], ref_padded[valid], atol=1e-5, rtol=1e-5)


def test_rms_norm_swap_on_cpu():
    from transformers.models.t5.modeling_t5 import T5LayerNorm

    torch.manual_seed(0)
    block = torch.nn.Sequential(torch.nn.Linear(32, 32), T5LayerNorm(32, eps=1e-6))
    with torch.no_grad():
        block[1].weight.uniform_(0.5, 1.5)
    x = torch.randn(4, 7, 32)
    ref = block(x)
    assert fused_rms_norm(block) == 1
    assert isinstance(block[1], onn.FusedRMSNorm) and block[1].eps == 1e-6
    assert torch.allclose(block(x), ref, atol=1e-6, rtol=1e-6)
    assert fused_rms_norm(block) == 0  # idempotent


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpt2_through_the_fused_kernels(device, dtype):
    m = tiny_gpt2().to(device).to(dtype).eval()
    ids, am = inputs()
    ids, am = ids.to(device), am.to(device)
    with torch.no_grad():
        ref_causal = m(ids).logits.float()
        ref_padded = m(ids, attention_mask=am).logits.float()
    fused_layer_norm(m)
    fused_scale_mask_softmax(m)
    with torch.no_grad():
        out_causal = m(ids).logits.float()
        out_padded = m(ids, attention_mask=am).logits.float()
    tol = 2e-4 if dtype == torch.float32 else 6e-2
    assert (out_causal - ref_causal).abs().max().item() <= tol
    valid = am.bool()
    assert (out_padded[valid] - ref_padded[valid]).abs().max().item() <= tol
    # generation with a key/value cache: one query against a growing key length
    with torch.no_grad():
        gen = m.generate(ids[:1, :8], max_new_tokens=6, do_sample=False)
    assert gen.shape == (1, 14)


@pytest.mark.gpu
def test_gpt2_gradients_through_the_fused_kernels(device):
    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    ref = tiny_gpt2(seed=3).to(device).train()
    fused = tiny_gpt2(seed=3).to(device).train()
    for mod in (ref, fused):  # dropout off: the two paths draw different masks
        for x in mod.modules():
            if isinstance(x, torch.nn.Dropout):
                x.p = 0.0
        mod.config.attn_pdrop = 0.0
    for blk in list(ref.transformer.h) + list(fused.transformer.h):
        if hasattr(blk.attn, "attn_dropout"):
            blk.attn.attn_dropout.p = 0.0
        if hasattr(blk.attn, "attention_dropout"):
            blk.attn.attention_dropout = 0.0
    fused_layer_norm(fused)
    fused_scale_mask_softmax(fused)
    lr = ref(ids, attention_mask=am, labels=ids).loss
    lf = fused(ids, attention_mask=am, labels=ids).loss
    assert abs(lr.item() - lf.item()) <= 1e-4
    lr.backward()
    lf.backward()
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.abs().max().item() + 1e-8
        assert (pr.grad - pf.grad).abs().max().item() <= 2e-3 * scale + 1e-6, n


@pytest.mark.gpu
def test_attention_dropout_in_training_mode_uses_the_fused_kernel(device):
    m = tiny_gpt2(attn_pdrop=0.5, resid_pdrop=0.0, embd_pdrop=0.0).to(device).to(torch.bfloat16).train()
    fused_scale_mask_softmax(m)
    ids, _ = inputs()
    ids = ids.to(device)
    gen = torch.cuda.default_generators[torch.device(device).index or 0]
    torch.manual_seed(5)
    off = gen.get_offset()
    a = m(ids).logits
    assert gen.get_offset() == off + 4 * 2  # one fused softmax-dropout per layer
    torch.manual_seed(5)
    b = m(ids).logits
    assert torch.equal(a, b)  # the mask is a function of the generator state
    c = m(ids).logits
    assert not torch.equal(a, c)
    m.eval()
    off = gen.get_offset()
    m(ids)
    assert gen.get_offset() == off
