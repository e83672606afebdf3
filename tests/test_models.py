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


def tiny_bert(seed=0, **kw):
    from transformers import BertConfig, BertModel

    cfg = BertConfig(num_hidden_layers=2, num_attention_heads=4, hidden_size=128,
                     intermediate_size=256, vocab_size=211, max_position_embeddings=128, **kw)
    torch.manual_seed(seed)
    m = BertModel(cfg)
    m.config._attn_implementation = "eager"
    return m


def test_bert_swaps_on_cpu_keep_the_model_output():
    # post-LN blocks, bidirectional attention with a key-padding mask
    # (modeling_bert.py:298-306, 343-346 of the reference)
    m = tiny_bert().eval()
    ids, am = inputs()
    ref = m(ids, attention_mask=am).last_hidden_state
    assert fused_layer_norm(m) == 5  # embeddings + 2 x (attention output, output)
    fused_scale_mask_softmax(m)
    out = m(ids, attention_mask=am).last_hidden_state
    valid = am.bool()
    assert torch.allclose(out[valid], ref[valid], atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bert_through_the_fused_kernels(device, dtype, monkeypatch):
    from oslo_amd.transformers import kernel_fusion_utils as kfu

    m = tiny_bert().to(device).to(dtype).eval()
    ids, am = inputs()
    ids, am = ids.to(device), am.to(device)
    with torch.no_grad():
        ref = m(ids, attention_mask=am).last_hidden_state.float()
    fused_layer_norm(m)
    fused_scale_mask_softmax(m)
    calls = []
    masked = kfu.onn_f.scaled_masked_softmax_dropout

    def counted(scores, hidden, *a, **k):
        calls.append((tuple(scores.shape), tuple(hidden.shape)))
        return masked(scores, hidden, *a, **k)

    monkeypatch.setattr(kfu.onn_f, "scaled_masked_softmax_dropout", counted)
    with torch.no_grad():
        out = m(ids, attention_mask=am).last_hidden_state.float()
    # one padding-masked softmax per layer, with a [b, 1, 1 or sq, sk] mask
    assert len(calls) == 2 and all(s == (3, 4, 48, 48) and h[0] == 3 and h[1] == 1 for s, h in calls)
    tol = 2e-4 if dtype == torch.float32 else 6e-2
    valid = am.bool()
    assert (out[valid] - ref[valid]).abs().max().item() <= tol


@pytest.mark.gpu
def test_bert_gradients_through_the_fused_kernels(device):
    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    kw = dict(hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    ref = tiny_bert(seed=3, **kw).to(device).train()
    fused = tiny_bert(seed=3, **kw).to(device).train()
    fused_layer_norm(fused)
    fused_scale_mask_softmax(fused)
    valid = am.bool()
    w = torch.randn(3, 32, 128, generator=torch.Generator().manual_seed(9)).to(device)
    lr = (ref(ids, attention_mask=am).last_hidden_state * w)[valid].sum()
    lf = (fused(ids, attention_mask=am).last_hidden_state * w)[valid].sum()
    assert abs(lr.item() - lf.item()) <= 1e-3 * (abs(lr.item()) + 1.0)
    lr.backward()
    lf.backward()
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.abs().max().item() + 1e-8
        assert (pr.grad - pf.grad).abs().max().item() <= 2e-3 * scale + 1e-6, n


def test_post_ln_output_swap_on_cpu_keeps_the_model_output():
    from oslo_amd.transformers import fused_bias_dropout_add_layer_norm

    m = tiny_bert().eval()
    ids, am = inputs()
    ref = m(ids, attention_mask=am).last_hidden_state
    fused_layer_norm(m)  # either order: the swap accepts both norm classes
    assert fused_bias_dropout_add_layer_norm(m) == 4  # 2 x (attention output, output)
    assert fused_bias_dropout_add_layer_norm(m) == 0  # idempotent
    assert type(m.encoder.layer[0].output).__name__ == "FusedBertOutput"
    out = m(ids, attention_mask=am).last_hidden_state
    assert torch.allclose(out, ref, atol=1e-5, rtol=1e-5)
    # a GPT-2 block has no post-LN output block
    assert fused_bias_dropout_add_layer_norm(tiny_gpt2()) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bert_post_ln_blocks_through_the_fused_kernel(device, dtype, monkeypatch):
    from oslo_amd.torch import _C
    from oslo_amd.transformers import fused_bias_dropout_add_layer_norm

    kw = dict(hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    ref = tiny_bert(seed=3, **kw).to(device).to(dtype).train()
    fused = tiny_bert(seed=3, **kw).to(device).to(dtype).train()
    assert fused_bias_dropout_add_layer_norm(fused) == 4
    fused_layer_norm(fused)
    fused_scale_mask_softmax(fused)
    kernel = _C.get_layernorm_kernel()
    calls = []
    fwd = kernel.bias_dropout_add_norm_forward

    def counted(*a, **k):
        calls.append(1)
        return fwd(*a, **k)

    monkeypatch.setattr(kernel, "bias_dropout_add_norm_forward", counted)
    valid = am.bool()
    w = torch.randn(3, 32, 128, generator=torch.Generator().manual_seed(9)).to(device).to(dtype)
    lr = (ref(ids, attention_mask=am).last_hidden_state * w)[valid].float().sum()
    lf = (fused(ids, attention_mask=am).last_hidden_state * w)[valid].float().sum()
    assert len(calls) == 4  # every post-LN block ran the one-kernel op
    tol = 1e-3 if dtype == torch.float32 else 5e-2
    assert abs(lr.item() - lf.item()) <= tol * (abs(lr.item()) + 1.0)
    lr.backward()
    lf.backward()
    gtol = 2e-3 if dtype == torch.float32 else 8e-2
    # (the key bias has a zero gradient, softmax being shift-invariant: in bf16
    #  what is left of it is rounding noise, hence the floor on the scale)
    gmax = max(p.grad.float().abs().max().item() for p in ref.parameters() if p.grad is not None)
    floor = 1e-8 if dtype == torch.float32 else 1e-3 * gmax
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.float().abs().max().item() + floor
        assert (pr.grad.float() - pf.grad.float()).abs().max().item() <= gtol * scale + 1e-6, n


@pytest.mark.gpu
def test_bert_post_ln_dropout_draws_from_the_generator(device):
    from oslo_amd.transformers import fused_bias_dropout_add_layer_norm

    m = tiny_bert(hidden_dropout_prob=0.3, attention_probs_dropout_prob=0.0).to(device).train()
    fused_bias_dropout_add_layer_norm(m)
    ids, am = inputs()
    ids, am = ids.to(device), am.to(device)
    torch.manual_seed(5)
    a = m(ids, attention_mask=am).last_hidden_state
    torch.manual_seed(5)
    b = m(ids, attention_mask=am).last_hidden_state
    assert torch.equal(a, b)
    c = m(ids, attention_mask=am).last_hidden_state
    assert not torch.equal(a, c)
    m.eval()
    d = m(ids, attention_mask=am).last_hidden_state
    e = m(ids, attention_mask=am).last_hidden_state
    assert torch.equal(d, e)


def test_bias_gelu_swap_on_cpu_keeps_the_model_output():
    from oslo_amd.transformers import fused_bias_gelu

    m = tiny_gpt2().eval()  # activation "gelu_new": the tanh form
    ids, am = inputs()
    ref = m(ids).logits
    assert fused_bias_gelu(m) == 2 and fused_bias_gelu(m) == 0
    assert type(m.transformer.h[0].mlp).__name__ == "FusedGPT2MLP"
    assert torch.allclose(m(ids).logits, ref, atol=1e-5, rtol=1e-5)
    # the erf form of GeLU is another function: such blocks stay as they are
    assert fused_bias_gelu(tiny_bert()) == 0
    b = tiny_bert(hidden_act="gelu_new").eval()
    ref = b(ids, attention_mask=am).last_hidden_state
    assert fused_bias_gelu(b) == 2
    assert torch.allclose(b(ids, attention_mask=am).last_hidden_state, ref, atol=1e-5, rtol=1e-5)


def test_bias_gelu_swap_with_the_tanh_form_for_the_exact_one():
    """The reference's models evaluate the tanh form whatever the configuration
    names (modeling_bert.py:426): the swap does the same on request, and the
    output then moves by what the two forms differ by (4.7e-4 at most per
    activation), no more."""
    from oslo_amd.transformers import fuse_all, fused_bias_gelu

    ids, am = inputs()
    b = tiny_bert().eval()   # "gelu": x * Phi(x)
    with torch.no_grad():
        ref = b(ids, attention_mask=am).last_hidden_state
    assert fused_bias_gelu(b) == 0
    assert fused_bias_gelu(b, tanh_for_erf=True) == 2 and fused_bias_gelu(b, tanh_for_erf=True) == 0
    with torch.no_grad():
        out = b(ids, attention_mask=am).last_hidden_state
    err = (out - ref).abs().max().item()
    assert 1e-6 < err < 2e-2, err   # another function, close to the first
    # a relu block is neither form
    import transformers as tf
    opt = tf.OPTForCausalLM(tf.OPTConfig(hidden_size=64, ffn_dim=128, num_hidden_layers=1, num_attention_heads=4,
                                         word_embed_proj_dim=64, vocab_size=211, max_position_embeddings=64))
    assert fuse_all(opt, attention=False, tanh_for_erf=True)["fused_bias_gelu"] == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpt2_with_every_swap_outputs_and_gradients(device, dtype, monkeypatch):
    from oslo_amd.torch import _C
    from oslo_amd.transformers import fused_bias_gelu

    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    kw = dict(attn_pdrop=0.0, resid_pdrop=0.0, embd_pdrop=0.0)
    ref = tiny_gpt2(seed=3, **kw).to(device).to(dtype).train()
    fused = tiny_gpt2(seed=3, **kw).to(device).to(dtype).train()
    assert fused_bias_gelu(fused) == 2
    fused_layer_norm(fused)
    fused_scale_mask_softmax(fused)
    kernel = _C.get_fused_elementwise_kernel()
    calls = []
    fwd = kernel.bias_gelu_forward

    def counted(*a, **k):
        calls.append(1)
        return fwd(*a, **k)

    monkeypatch.setattr(kernel, "bias_gelu_forward", counted)
    lr = ref(ids, attention_mask=am, labels=ids).loss
    lf = fused(ids, attention_mask=am, labels=ids).loss
    assert len(calls) == 2  # one bias-GeLU kernel per block
    assert abs(lr.item() - lf.item()) <= (1e-4 if dtype == torch.float32 else 3e-2)
    lr.backward()
    lf.backward()
    gtol = 2e-3 if dtype == torch.float32 else 8e-2
    gmax = max(p.grad.float().abs().max().item() for p in ref.parameters() if p.grad is not None)
    floor = 1e-8 if dtype == torch.float32 else 1e-3 * gmax
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.float().abs().max().item() + floor
        assert (pr.grad.float() - pf.grad.float()).abs().max().item() <= gtol * scale + 1e-6, n


def test_pre_ln_block_swap_on_cpu_keeps_the_model_output():
    from oslo_amd.transformers import fused_bias_gelu, fused_pre_ln_block

    ids, am = inputs()
    for gelu_first in (False, True):
        m = tiny_gpt2().eval()
        ref, ref_padded = m(ids).logits, m(ids, attention_mask=am).logits
        keys = list(m.state_dict())
        if gelu_first:
            assert fused_bias_gelu(m) == 2
        assert fused_pre_ln_block(m) == 2 and fused_pre_ln_block(m) == 0
        if not gelu_first:
            assert fused_bias_gelu(m) == 2
        assert list(m.state_dict()) == keys  # checkpoints keep loading
        assert torch.allclose(m(ids).logits, ref, atol=1e-5, rtol=1e-5)
        valid = am.bool()
        assert torch.allclose(m(ids, attention_mask=am).logits[valid], ref_padded[valid], atol=1e-5, rtol=1e-5)
        gen = m.generate(ids[:1, :8], max_new_tokens=4, do_sample=False)
        assert gen.shape == (1, 12)
    assert fused_pre_ln_block(tiny_bert()) == 0  # post-LN blocks are another shape


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpt2_pre_ln_blocks_through_the_fused_kernels(device, dtype, monkeypatch):
    from oslo_amd.torch import _C
    from oslo_amd.transformers import fused_bias_gelu, fused_pre_ln_block

    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    kw = dict(attn_pdrop=0.0, resid_pdrop=0.0, embd_pdrop=0.0)
    ref = tiny_gpt2(seed=3, **kw).to(device).to(dtype).train()
    fused = tiny_gpt2(seed=3, **kw).to(device).to(dtype).train()
    assert fused_pre_ln_block(fused) == 2
    fused_bias_gelu(fused)
    fused_layer_norm(fused)
    fused_scale_mask_softmax(fused)
    norm_kernel, elt_kernel = _C.get_layernorm_kernel(), _C.get_fused_elementwise_kernel()
    calls = []
    norm_fwd, bda_fwd = norm_kernel.bias_dropout_add_norm_forward, elt_kernel.bias_dropout_add_forward
    monkeypatch.setattr(norm_kernel, "bias_dropout_add_norm_forward",
                        lambda *a, **k: (calls.append("norm"), norm_fwd(*a, **k))[1])
    monkeypatch.setattr(elt_kernel, "bias_dropout_add_forward",
                        lambda *a, **k: (calls.append("bda"), bda_fwd(*a, **k))[1])
    lr = ref(ids, attention_mask=am, labels=ids).loss
    lf = fused(ids, attention_mask=am, labels=ids).loss
    assert calls == ["norm", "bda"] * 2  # per block: residual add inside ln_2, then the MLP's
    assert abs(lr.item() - lf.item()) <= (1e-4 if dtype == torch.float32 else 3e-2)
    lr.backward()
    lf.backward()
    gtol = 2e-3 if dtype == torch.float32 else 8e-2
    gmax = max(p.grad.float().abs().max().item() for p in ref.parameters() if p.grad is not None)
    floor = 1e-8 if dtype == torch.float32 else 1e-3 * gmax
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.float().abs().max().item() + floor
        assert (pr.grad.float() - pf.grad.float()).abs().max().item() <= gtol * scale + 1e-6, n


@pytest.mark.gpu
def test_gpt2_pre_ln_residual_dropout_draws_from_the_generator(device):
    from oslo_amd.transformers import fused_pre_ln_block

    m = tiny_gpt2(attn_pdrop=0.0, resid_pdrop=0.3, embd_pdrop=0.0).to(device).train()
    assert fused_pre_ln_block(m) == 2
    ids, _ = inputs()
    ids = ids.to(device)
    gen = torch.cuda.default_generators[torch.device(device).index or 0]
    torch.manual_seed(7)
    off = gen.get_offset()
    a = m(ids).logits
    assert gen.get_offset() == off + 4 * 4  # two fused dropouts per block
    torch.manual_seed(7)
    b = m(ids).logits
    assert torch.equal(a, b)
    assert not torch.equal(a, m(ids).logits)
    m.eval()
    assert torch.equal(m(ids).logits, m(ids).logits)


def test_fuse_all_on_cpu():
    from oslo_amd.transformers import fuse_all

    ids, am = inputs()
    m = tiny_gpt2().eval()
    ref = m(ids, attention_mask=am).logits
    assert fuse_all(m) == {
        "fused_pre_ln_block": 2, "fused_bias_dropout_add_layer_norm": 0, "fused_bias_gelu": 2,
        "fused_layer_norm": 5, "fused_rms_norm": 0, "fused_scale_mask_softmax": True,
    }
    valid = am.bool()
    assert torch.allclose(m(ids, attention_mask=am).logits[valid], ref[valid], atol=1e-5, rtol=1e-5)
    b = tiny_bert().eval()
    ref = b(ids, attention_mask=am).last_hidden_state
    changed = fuse_all(b)
    assert changed["fused_bias_dropout_add_layer_norm"] == 4 and changed["fused_layer_norm"] == 5
    assert changed["fused_pre_ln_block"] == 0 and changed["fused_bias_gelu"] == 0
    assert torch.allclose(b(ids, attention_mask=am).last_hidden_state[valid], ref[valid], atol=1e-5, rtol=1e-5)


def tiny_neox(seed=0, **kw):
    from transformers import GPTNeoXConfig, GPTNeoXForCausalLM

    torch.manual_seed(seed)
    cfg = GPTNeoXConfig(vocab_size=211, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                        intermediate_size=256, hidden_act="gelu_fast", max_position_embeddings=64,
                        use_parallel_residual=True, attention_dropout=0.0, hidden_dropout=0.0, **kw)
    return GPTNeoXForCausalLM(cfg)


def test_gpt_neox_swaps_on_cpu_keep_the_model_output():
    """The GPT-NeoX block (the shape of BASELINE configuration 5): its MLP has
    no dropout of its own and names its projections dense_h_to_4h /
    dense_4h_to_h; norms, bias-GeLU and the attention function are swapped."""
    from oslo_amd.transformers import fuse_all

    ids, am = inputs()
    m = tiny_neox().eval()
    ref = m(ids, attention_mask=am).logits
    changed = fuse_all(m)
    assert changed["fused_bias_gelu"] == 2 and changed["fused_layer_norm"] == 5
    assert changed["fused_scale_mask_softmax"] is True
    valid = am.bool()
    assert torch.allclose(m(ids, attention_mask=am).logits[valid], ref[valid], atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpt_neox_with_every_swap_outputs_and_gradients(device, dtype, monkeypatch):
    from oslo_amd.torch import _C
    from oslo_amd.transformers import fuse_all

    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    ref = tiny_neox(seed=5).to(device).to(dtype).train()
    fused = tiny_neox(seed=5).to(device).to(dtype).train()
    changed = fuse_all(fused)
    assert changed["fused_bias_gelu"] == 2 and changed["fused_layer_norm"] == 5
    kernel = _C.get_fused_elementwise_kernel()
    sm = _C.get_softmax_kernel()
    calls = {"gelu": 0, "softmax": 0}
    gelu_fwd, sm_fwd = kernel.bias_gelu_forward, sm.fused_scaled_masked_softmax_forward

    def counted_gelu(*a, **k):
        calls["gelu"] += 1
        return gelu_fwd(*a, **k)

    def counted_softmax(*a, **k):
        calls["softmax"] += 1
        return sm_fwd(*a, **k)

    monkeypatch.setattr(kernel, "bias_gelu_forward", counted_gelu)
    monkeypatch.setattr(sm, "fused_scaled_masked_softmax_forward", counted_softmax)
    lr = ref(ids, attention_mask=am, labels=ids).loss
    lf = fused(ids, attention_mask=am, labels=ids).loss
    assert calls["gelu"] == 2      # one bias-GeLU kernel per block
    assert calls["softmax"] == 2   # a padded causal batch: the masked softmax kernel, once per block
    assert abs(lr.item() - lf.item()) <= (1e-4 if dtype == torch.float32 else 3e-2)
    lr.backward()
    lf.backward()
    gtol = 2e-3 if dtype == torch.float32 else 8e-2
    gmax = max(p.grad.float().abs().max().item() for p in ref.parameters() if p.grad is not None)
    floor = 1e-8 if dtype == torch.float32 else 1e-3 * gmax
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.float().abs().max().item() + floor
        assert (pr.grad.float() - pf.grad.float()).abs().max().item() <= gtol * scale + 1e-6, n


def _family(name):
    import transformers as tf

    kw = dict(vocab_size=211, max_position_embeddings=64)
    if name == "llama":
        return tf.LlamaForCausalLM(tf.LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                                  num_attention_heads=4, num_key_value_heads=2, **kw))
    if name == "mistral":
        return tf.MistralForCausalLM(tf.MistralConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                                      num_attention_heads=4, num_key_value_heads=2,
                                                      sliding_window=16, **kw))
    if name == "gptj":
        return tf.GPTJForCausalLM(tf.GPTJConfig(vocab_size=211, n_embd=64, n_layer=2, n_head=4, rotary_dim=8,
                                                n_positions=64))
    if name == "opt":
        return tf.OPTForCausalLM(tf.OPTConfig(hidden_size=64, ffn_dim=128, num_hidden_layers=2,
                                              num_attention_heads=4, word_embed_proj_dim=64, dropout=0.0, **kw))
    if name == "bloom":
        return tf.BloomForCausalLM(tf.BloomConfig(vocab_size=211, hidden_size=64, n_layer=2, n_head=4))
    raise ValueError(name)


# what fuse_all finds in each architecture: (layer norms, rms norms, bias-GeLU blocks, attention swapped)
FAMILIES = {
    "llama": (0, 5, 0, True),      # RMSNorm, grouped-query attention
    "mistral": (0, 5, 0, True),    # sliding-window mask: the general masked kernel
    "gptj": (3, 0, 2, False),      # fc_in / fc_out MLP with gelu_new
    "opt": (5, 0, 0, True),
    "bloom": (6, 0, 0, False),
}


@pytest.mark.parametrize("name", sorted(FAMILIES))
def test_fuse_all_across_architectures_on_cpu(name):
    from oslo_amd.transformers import fuse_all

    torch.manual_seed(0)
    m = _family(name).eval()
    ids, am = inputs()
    with torch.no_grad():
        ref = m(ids, attention_mask=am).logits
    changed = fuse_all(m)
    ln, rms, gelu, attn = FAMILIES[name]
    assert (changed["fused_layer_norm"], changed["fused_rms_norm"], changed["fused_bias_gelu"],
            changed["fused_scale_mask_softmax"]) == (ln, rms, gelu, attn), changed
    with torch.no_grad():
        out = m(ids, attention_mask=am).logits
    valid = am.bool()
    assert torch.allclose(out[valid], ref[valid], atol=2e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["llama", "mistral", "gptj", "opt"])
def test_fuse_all_across_architectures_on_gpu(device, name):
    """Logits and every parameter gradient of the swapped model against the
    model as Hugging Face builds it, fp32, on a right-padded batch."""
    from oslo_amd.transformers import fuse_all

    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    torch.manual_seed(0)
    ref = _family(name).to(device).train()
    torch.manual_seed(0)
    fused = _family(name).to(device).train()
    fuse_all(fused)
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


def tiny_bart(seed=0):
    from transformers import BartConfig, BartForConditionalGeneration

    cfg = BartConfig(vocab_size=211, d_model=64, encoder_layers=2, decoder_layers=2, encoder_attention_heads=4,
                     decoder_attention_heads=4, encoder_ffn_dim=128, decoder_ffn_dim=128,
                     max_position_embeddings=64, dropout=0.0, attention_dropout=0.0, activation_dropout=0.0)
    torch.manual_seed(seed)
    return BartForConditionalGeneration(cfg)


def bart_inputs(seed=1):
    g = torch.Generator().manual_seed(seed)
    src = torch.randint(3, 211, (3, 24), generator=g)
    am = torch.ones(3, 24, dtype=torch.long)
    am[1, 17:] = 0
    am[2, 9:] = 0
    return src, am, torch.randint(3, 211, (3, 10), generator=g)


def test_bart_swaps_on_cpu_keep_the_model_output():
    """An encoder-decoder in the layout of oslo/transformers/models/bart/modeling_bart.py:
    padded encoder self-attention, causal decoder self-attention, cross-attention of 10
    queries over 24 padded keys."""
    from oslo_amd.transformers import fuse_all

    m = tiny_bart().eval()
    src, am, dec = bart_inputs()
    with torch.no_grad():
        ref = m(input_ids=src, attention_mask=am, decoder_input_ids=dec).logits
    changed = fuse_all(m)
    assert changed["fused_scale_mask_softmax"] and changed["fused_layer_norm"] == 12
    with torch.no_grad():
        out = m(input_ids=src, attention_mask=am, decoder_input_ids=dec).logits
    assert torch.allclose(out, ref, atol=2e-5, rtol=1e-5)


@pytest.mark.gpu
def test_bart_through_the_fused_kernels(device, monkeypatch):
    """Loss and every parameter gradient, fp32; the three kinds of attention reach
    the padding-masked, the causal and (cross-attention, sq != sk) the padding-masked
    kernel again, none of them the unfused chain."""
    import warnings

    from oslo_amd.transformers import fuse_all

    masked = _spy(monkeypatch, "scaled_masked_softmax_dropout")
    causal = _spy(monkeypatch, "scaled_upper_triang_masked_softmax_dropout")
    src, am, dec = (t.to(device) for t in bart_inputs())
    ref = tiny_bart().to(device).train()
    fused = tiny_bart().to(device).train()
    fuse_all(fused)
    lr = ref(input_ids=src, attention_mask=am, decoder_input_ids=dec, labels=dec).loss
    with warnings.catch_warnings():
        warnings.simplefilter("error", RuntimeWarning)   # the unfused chain would warn
        lf = fused(input_ids=src, attention_mask=am, decoder_input_ids=dec, labels=dec).loss
    assert abs(lr.item() - lf.item()) <= 1e-4
    # 2 encoder layers + 2 cross-attentions with the source's padding mask; 2 causal decoder layers
    assert len(masked) + len(causal) == 6 and len(causal) >= 2, (len(masked), len(causal))
    lr.backward()
    lf.backward()
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.abs().max().item() + 1e-8
        assert (pr.grad - pf.grad).abs().max().item() <= 2e-3 * scale + 1e-6, n


# The encoder families the reference ships next to BERT, GPT-2, BART and T5
# (oslo/transformers/models/{distilbert,roberta,albert,electra,mbart,mt5}), as Hugging Face builds them today.
def _reference_family(name, seed=0):
    import transformers as tf

    kw = dict(vocab_size=211, max_position_embeddings=64)
    enc = dict(hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
               hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    torch.manual_seed(seed)
    if name == "distilbert":   # masked_fill(mask == 0, -inf): modeling_distilbert.py:225-234
        return tf.DistilBertForMaskedLM(tf.DistilBertConfig(dim=64, hidden_dim=128, n_layers=2, n_heads=4,
                                                            dropout=0.0, attention_dropout=0.0, **kw))
    if name == "roberta":
        return tf.RobertaForMaskedLM(tf.RobertaConfig(**enc, **kw))
    if name == "albert":
        return tf.AlbertForMaskedLM(tf.AlbertConfig(embedding_size=32, **enc, **kw))
    if name == "electra":
        return tf.ElectraForMaskedLM(tf.ElectraConfig(embedding_size=32, **enc, **kw))
    if name == "mbart":
        return tf.MBartForConditionalGeneration(tf.MBartConfig(
            d_model=64, encoder_layers=2, decoder_layers=2, encoder_attention_heads=4, decoder_attention_heads=4,
            encoder_ffn_dim=128, decoder_ffn_dim=128, dropout=0.0, attention_dropout=0.0, activation_dropout=0.0,
            **kw))
    if name == "mt5":
        return tf.MT5ForConditionalGeneration(tf.MT5Config(vocab_size=211, d_model=64, d_kv=16, d_ff=128,
                                                           num_layers=2, num_decoder_layers=2, num_heads=4,
                                                           dropout_rate=0.0, decoder_start_token_id=0,
                                                           pad_token_id=0))
    raise ValueError(name)


# (layer norms, rms norms, post-LN output blocks, softmax kernel launches of one forward pass)
REFERENCE_FAMILIES = {
    "distilbert": (6, 0, 0, 2),
    "roberta": (6, 0, 4, 2),
    "albert": (4, 0, 0, 2),     # one shared layer, run twice
    "electra": (6, 0, 4, 2),
    "mbart": (14, 0, 0, 6),     # encoder, decoder self- and cross-attention
    "mt5": (0, 12, 0, 6),
}


def _family_call(name, m, src, am, dec, labels=False):
    kw = dict(input_ids=src, attention_mask=am)
    if name in ("mbart", "mt5"):
        kw["decoder_input_ids"] = dec
        if labels:
            kw["labels"] = dec
    elif labels:
        kw["labels"] = src
    return m(**kw)


@pytest.mark.parametrize("name", sorted(REFERENCE_FAMILIES))
def test_reference_families_on_cpu(name):
    from oslo_amd.transformers import fuse_all

    m = _reference_family(name).eval()
    src, am, dec = bart_inputs()
    with torch.no_grad():
        ref = _family_call(name, m, src, am, dec).logits
    changed = fuse_all(m)
    ln, rms, post_ln, _ = REFERENCE_FAMILIES[name]
    assert (changed["fused_layer_norm"], changed["fused_rms_norm"],
            changed["fused_bias_dropout_add_layer_norm"], changed["fused_scale_mask_softmax"]) == \
        (ln, rms, post_ln, True), changed
    with torch.no_grad():
        out = _family_call(name, m, src, am, dec).logits
    if name not in ("mbart", "mt5"):   # (the rows of padding tokens attend to nothing meaningful)
        out, ref = out[am.bool()], ref[am.bool()]
    assert torch.allclose(out, ref, atol=5e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(REFERENCE_FAMILIES))
def test_reference_families_through_the_fused_kernels(device, monkeypatch, name):
    """Loss and every parameter gradient of the swapped model against the model
    as Hugging Face builds it, fp32, on a right-padded batch; every attention
    of the forward pass reaches a softmax kernel and none the unfused chain."""
    import warnings

    from oslo_amd.transformers import fuse_all

    spies = [_spy(monkeypatch, fn) for fn in ("scaled_masked_softmax_dropout",
                                              "scaled_upper_triang_masked_softmax_dropout",
                                              "scaled_bias_softmax_dropout")]
    src, am, dec = (t.to(device) for t in bart_inputs())
    ref = _reference_family(name).to(device).train()
    fused = _reference_family(name).to(device).train()
    fuse_all(fused)
    lr = _family_call(name, ref, src, am, dec, labels=True).loss
    with warnings.catch_warnings():
        warnings.simplefilter("error", RuntimeWarning)   # the unfused chain would warn
        lf = _family_call(name, fused, src, am, dec, labels=True).loss
    assert abs(lr.item() - lf.item()) <= 1e-4 * max(1.0, abs(lr.item()))
    assert sum(len(s) for s in spies) == REFERENCE_FAMILIES[name][3], [len(s) for s in spies]
    lr.backward()
    lf.backward()
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.abs().max().item() + 1e-8
        assert (pr.grad - pf.grad).abs().max().item() <= 2e-3 * scale + 1e-6, n


def tiny_t5(seed=0):
    from transformers import T5Config, T5ForConditionalGeneration

    cfg = T5Config(d_model=128, d_kv=32, d_ff=256, num_layers=2, num_decoder_layers=2, num_heads=4,
                   vocab_size=211, decoder_start_token_id=0, pad_token_id=0, dropout_rate=0.0)
    torch.manual_seed(seed)
    return T5ForConditionalGeneration(cfg)


def t5_inputs(seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(1, 211, (3, 24), generator=g), torch.randint(1, 211, (3, 10), generator=g)


def test_t5_rms_norm_swap_on_cpu_keeps_the_model_output():
    # the swap the reference ships (kernel_fusion_utils.py:71-87), on a whole model
    m = tiny_t5().eval()
    ids, labels = t5_inputs()
    ref = m(input_ids=ids, labels=labels).logits
    assert fused_rms_norm(m) == 12  # encoder 2 x 2 + 1, decoder 2 x 3 + 1
    assert torch.allclose(m(input_ids=ids, labels=labels).logits, ref, atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_t5_through_the_fused_rms_norm(device, dtype):
    ids, labels = t5_inputs()
    ids, labels = ids.to(device), labels.to(device)
    ref = tiny_t5(seed=2).to(device).to(dtype).train()
    fused = tiny_t5(seed=2).to(device).to(dtype).train()
    assert fused_rms_norm(fused) == 12
    lr = ref(input_ids=ids, labels=labels).loss
    lf = fused(input_ids=ids, labels=labels).loss
    assert abs(lr.item() - lf.item()) <= (1e-4 if dtype == torch.float32 else 5e-2)
    lr.backward()
    lf.backward()
    gtol = 2e-3 if dtype == torch.float32 else 1e-1
    gmax = max(p.grad.float().abs().max().item() for p in ref.parameters() if p.grad is not None)
    floor = 1e-8 if dtype == torch.float32 else 2e-3 * gmax
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        scale = pr.grad.float().abs().max().item() + floor
        assert (pr.grad.float() - pf.grad.float()).abs().max().item() <= gtol * scale + 1e-6, n


def _eager_everywhere(model):
    for module in model.modules():
        if hasattr(module, "config") and hasattr(module.config, "_attn_implementation"):
            module.config._attn_implementation = "eager"
    return model


def test_t5_attention_reaches_the_registered_function_on_cpu():
    """T5's stacks hold their own configuration copies: the swap has to reach
    them, and every attention of the model (encoder with a padding mask,
    causal decoder, cross attention) then runs through the registered function
    with its position bias."""
    m = _eager_everywhere(tiny_t5()).eval()
    ids, labels = t5_inputs()
    am = torch.ones_like(ids)
    am[1, 18:] = 0
    ref = m(input_ids=ids, attention_mask=am, labels=labels).logits
    fused_scale_mask_softmax(m)
    att = m.encoder.block[0].layer[0].SelfAttention
    assert att.config._attn_implementation == m.decoder.config._attn_implementation == "oslo_fused_softmax"
    out = m(input_ids=ids, attention_mask=am, labels=labels).logits
    assert torch.allclose(out, ref, atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("padded", [False, True])
def test_t5_through_the_additive_term_softmax(device, dtype, padded, monkeypatch):
    """The model the reference's kernel_fusion_utils.py:71-87 fuses, with its
    attention (scores + position bias + mask, modeling_t5.py:508-514) through
    softmax(scale * x + term) and its norms through the RMS-norm swap: loss
    and every parameter gradient, the learned relative-attention bias included
    (its gradient is the gradient of the term summed over the batch)."""
    calls = _spy(monkeypatch, "scaled_bias_softmax_dropout")
    ids, labels = t5_inputs()
    am = torch.ones_like(ids)
    if padded:
        am[1, 18:] = 0
        am[2, 9:] = 0
    ids, labels, am = ids.to(device), labels.to(device), am.to(device)
    # the same (rounded) parameters evaluated in float32, eager
    truth = _eager_everywhere(tiny_t5(seed=2)).to(device).to(dtype).float().train()
    ref = _eager_everywhere(tiny_t5(seed=2)).to(device).to(dtype).train()   # eager in `dtype`
    fused = _eager_everywhere(tiny_t5(seed=2)).to(device).to(dtype).train()
    fused_scale_mask_softmax(fused)
    assert fused_rms_norm(fused) == 12
    lt = truth(input_ids=ids, attention_mask=am, labels=labels).loss
    lr = ref(input_ids=ids, attention_mask=am, labels=labels).loss
    lf = fused(input_ids=ids, attention_mask=am, labels=labels).loss
    assert len(calls) == 6  # 2 encoder + 2 decoder self + 2 cross attentions
    assert abs(lt.item() - lf.item()) <= (1e-4 if dtype == torch.float32 else 5e-2)
    for loss in (lt, lr, lf):
        loss.backward()
    # float32: the fused model against the eager one.  bfloat16: two bfloat16 models differ
    # by their rounding noise, so each is measured against the float32 model and the fused
    # one must not be further from it than the eager one (plus a floor).
    names = []
    for (n, pt), (_, pr), (_, pf) in zip(truth.named_parameters(), ref.named_parameters(),
                                         fused.named_parameters()):
        if pt.grad is None:
            continue
        names.append(n)
        scale = pt.grad.abs().max().item() + 1e-8
        err_f = (pf.grad.float() - pt.grad).abs().max().item()
        if dtype == torch.float32:
            assert err_f <= 2e-3 * scale + 1e-6, n
        else:
            err_r = (pr.grad.float() - pt.grad).abs().max().item()
            assert err_f <= 2.0 * err_r + 2e-2 * scale, (n, err_f, err_r, scale)
    assert any("relative_attention_bias" in n for n in names)


# ---------------------------------------------------------------------------
# the attention function registered with transformers: masks it may be handed
# ---------------------------------------------------------------------------
class _AttnStub(torch.nn.Module):
    def __init__(self, is_causal):
        super().__init__()
        self.is_causal = is_causal


def _eager_attention(q, k, v, scaling, additive):
    t = torch.matmul(q, k.transpose(-1, -2)) * scaling
    if additive is not None:
        t = t + additive
    return torch.matmul(torch.softmax(t, dim=-1), v).transpose(1, 2)


def _t5_style_bias(heads, sq, sk, seed):
    """A finite relative-position bias per head plus a -10000 key-padding fill,
    the sum T5 hands to its attention
    (oslo/transformers/models/t5/modeling_t5.py:508-514)."""
    g = torch.Generator().manual_seed(seed)
    rel = torch.randn(heads, 2 * max(sq, sk) - 1, generator=g)
    idx = torch.arange(sk)[None, :] - torch.arange(sq)[:, None] + max(sq, sk) - 1
    bias = rel[:, idx].unsqueeze(0)                      # [1, heads, sq, sk]
    pad = torch.zeros(2, 1, 1, sk)
    pad[1, ..., sk - 5:] = -10000.0
    return bias + pad                                    # [2, heads, sq, sk]


def test_additive_float_mask_is_applied_not_dropped_cpu():
    from oslo_amd.transformers.kernel_fusion_utils import fused_attention_forward

    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 4, 24, 16, generator=g) for _ in range(3))
    bias = _t5_style_bias(4, 24, 24, seed=1)
    out, _ = fused_attention_forward(_AttnStub(False).eval(), q, k, v, bias, scaling=1.0)
    assert torch.allclose(out, _eager_attention(q, k, v, 1.0, bias), rtol=1e-5, atol=1e-6)


def _spy(monkeypatch, name):
    """Records the calls of oslo_amd.torch.nn.modules.functional.<name>."""
    from oslo_amd.torch.nn.modules import functional as onn_f

    calls = []
    real = getattr(onn_f, name)

    def spy(*args, **kwargs):
        calls.append((args, kwargs))
        return real(*args, **kwargs)

    monkeypatch.setattr(onn_f, name, spy)
    return calls


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_additive_float_mask_takes_the_additive_term_kernel(device, dtype, monkeypatch):
    """A relative-position bias plus a -10000 fill is a finite additive term:
    it goes to the kernel that computes softmax(scale * x + term) and gives the
    eager result (a float mask must never be turned into a boolean one: the
    finite part would be lost)."""
    from oslo_amd.transformers.kernel_fusion_utils import fused_attention_forward

    calls = _spy(monkeypatch, "scaled_bias_softmax_dropout")
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 4, 24, 16, generator=g).to(device, dtype) for _ in range(3))
    bias = _t5_style_bias(4, 24, 24, seed=1).to(device, dtype)
    out, _ = fused_attention_forward(_AttnStub(False).eval(), q, k, v, bias, scaling=1.0)
    assert len(calls) == 1
    ref = _eager_attention(q.float(), k.float(), v.float(), 1.0, bias.float())
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert (out.float() - ref).abs().max().item() <= tol * (ref.abs().max().item() + 1.0)
    # and it is not what dropping the finite part would give
    dropped = _eager_attention(q.float(), k.float(), v.float(), 1.0,
                               torch.where(bias.float() < -1.0, -10000.0, 0.0))
    assert (out.float() - dropped).abs().max().item() > 10 * tol
    # the reference's own mask conventions, [b, 1, 1, sk]: (1 - m) * -10000
    # (modeling_bert.py:298-306) and finfo.min (modeling_bart.py:123-136)
    for fill in (-10000.0, torch.finfo(dtype).min):
        pad = torch.zeros(2, 1, 1, 24, device=device, dtype=dtype)
        pad[1, ..., 19:] = fill
        out, _ = fused_attention_forward(_AttnStub(False).eval(), q, k, v, pad, scaling=0.25)
        ref = _eager_attention(q.float(), k.float(), v.float(), 0.25, pad.float())
        assert (out.float() - ref).abs().max().item() <= tol * (ref.abs().max().item() + 1.0)
    assert len(calls) == 3
    # a separate position bias next to a boolean mask (the arguments T5 passes)
    rel = _t5_style_bias(4, 24, 24, seed=2)[:1].to(device, dtype)
    attend = torch.ones(2, 1, 24, 24, dtype=torch.bool, device=device)
    attend[1, ..., 17:] = False
    out, _ = fused_attention_forward(_AttnStub(False).eval(), q, k, v, attend, scaling=1.0,
                                     position_bias=rel)
    ref = _eager_attention(q.float(), k.float(), v.float(), 1.0,
                           rel.float() + torch.where(attend, 0.0, -10000.0))
    assert (out.float() - ref).abs().max().item() <= tol * (ref.abs().max().item() + 1.0)
    assert len(calls) == 4


def _attention_branch_cases(device):
    """(name, is_causal, sq, sk, mask, position_bias, kwargs, hidden [b or 1, h or 1, sq, sk] or None)"""
    from oslo_amd.transformers.kernel_fusion_utils import CausalKeyPaddingMask

    b, h, sq, sk = 2, 4, 12, 24
    g = torch.Generator().manual_seed(3)
    rel = torch.randn(1, h, sq, sk, generator=g).to(device)
    tri = torch.ones(sq, sk, dtype=torch.bool).tril(sk - sq).to(device)       # True = attend
    kv = torch.ones(b, sk, dtype=torch.bool, device=device)
    kv[1, sk - 5:] = False
    full = tri[None, None] & kv[:, None, None, :]
    cases = [
        ("no scaling given", True, sq, sk, None, None, {}, ~tri[None, None]),
        ("a layer that is not causal, without a mask", False, sq, sk, None, None, {}, None),
        ("is_causal given with the call", True, sq, sk, None, None, {"is_causal": False}, None),
        ("one query against its cache next to a position bias", True, 1, sk, None, rel[:, :, :1], {}, None),
        ("a mask longer than the keys", False, sq, sk, torch.cat([kv, kv], dim=1)[:, None, None, :], None, {},
         ~kv[:, None, None, :].expand(b, 1, sq, sk)),
        ("an integer mask", False, sq, sk, kv[:, None, None, :].to(torch.int64), None, {},
         ~kv[:, None, None, :].expand(b, 1, sq, sk)),
        ("a mask of three dimensions", False, sq, sk, tri[None], None, {}, ~tri[None, None]),
        ("a float mask next to a position bias", False, sq, sk,
         torch.where(kv, 0.0, -10000.0)[:, None, None, :], rel, {}, ~kv[:, None, None, :].expand(b, 1, sq, sk)),
        ("the causal key-padding mask next to a position bias", True, sq, sk,
         CausalKeyPaddingMask.wrap(full, kv), rel, {}, ~full),
    ]
    return cases, (b, h)


@pytest.mark.gpu
def test_every_branch_of_the_attention_function(device):
    """The calls the model tests do not make: default scaling, a call-time
    is_causal, decoding one query with a position bias, masks longer than the
    keys, integer and three-dimensional masks, a float mask or the causal
    key-padding mask next to a position bias;
    each against the eager chain on the same operands."""
    import warnings

    from oslo_amd.transformers.kernel_fusion_utils import fused_attention_forward

    cases, (b, h) = _attention_branch_cases(device)
    for name, is_causal, sq, sk, mask, bias, kwargs, hidden in cases:
        g = torch.Generator().manual_seed(len(name))
        q = torch.randn(b, h, sq, 16, generator=g).to(device)
        k, v = (torch.randn(b, h, sk, 16, generator=g).to(device) for _ in range(2))
        with warnings.catch_warnings():
            warnings.simplefilter("error", RuntimeWarning)   # the unfused chain would warn
            out, _ = fused_attention_forward(_AttnStub(is_causal).eval(), q, k, v, mask, position_bias=bias,
                                             **kwargs)
        additive = torch.zeros(1, 1, sq, sk, device=device)
        if bias is not None:
            additive = additive + bias
        if hidden is not None:
            additive = additive.expand(b, h, sq, sk).masked_fill(hidden.expand(b, h, sq, sk), float("-inf"))
        ref = _eager_attention(q, k, v, 16 ** -0.5, additive)
        assert (out - ref).abs().max().item() <= 2e-5 * (ref.abs().max().item() + 1.0), name


@pytest.mark.gpu
def test_boolean_mask_per_head_becomes_an_additive_term(device, monkeypatch):
    """The mask kernels broadcast one mask over the heads; a boolean mask that
    differs from head to head goes to the additive-term kernel as a fill that
    absorbs the logit."""
    from oslo_amd.transformers.kernel_fusion_utils import fused_attention_forward

    calls = _spy(monkeypatch, "scaled_bias_softmax_dropout")
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(2, 4, 24, 16, generator=g).to(device) for _ in range(3))
    attend = torch.rand(2, 4, 24, 24, generator=g) > 0.3
    attend[..., 0] = True  # every query sees a key
    out, _ = fused_attention_forward(_AttnStub(False).eval(), q, k, v, attend.to(device), scaling=0.25)
    additive = torch.where(attend, 0.0, -10000.0).to(device)
    ref = _eager_attention(q, k, v, 0.25, additive)
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    assert len(calls) == 1


@pytest.mark.gpu
def test_unfused_chain_on_the_gpu_warns_once(device):
    """A call the kernels cannot take (a mask on another device) runs the torch
    chain and says so, once per reason."""
    import warnings

    from oslo_amd.transformers import kernel_fusion_utils as kfu

    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(2, 4, 8, 16, generator=g).to(device).double() for _ in range(3))
    kfu._warned.clear()
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        for _ in range(3):
            out, _ = kfu.fused_attention_forward(_AttnStub(False).eval(), q, k, v, None, scaling=0.25,
                                                 is_causal=False)
    assert len([w for w in seen if "unfused torch chain" in str(w.message)]) == 1
    assert torch.allclose(out, _eager_attention(q, k, v, 0.25, None))
    # the module: a mask whose size does not broadcast is a reason, too
    from oslo_amd.torch.nn.modules.softmax import FusedScaleMaskSoftmax

    FusedScaleMaskSoftmax._warned.clear()
    m = FusedScaleMaskSoftmax(scale=0.5)
    x = torch.randn(2, 3, 4, 8, device=device, dtype=torch.float64)
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        m(x, None)
        m(x, None)
    assert len([w for w in seen if "unfused torch chain" in str(w.message)]) == 1


def test_mask_builder_returns_the_full_mask_and_the_key_part():
    from transformers import masking_utils as mu

    from oslo_amd.transformers.kernel_fusion_utils import fused_attention_mask, key_visible_of

    am = torch.ones(3, 20, dtype=torch.long)
    am[1, 15:] = 0
    am[2, :4] = 0
    full = fused_attention_mask(3, 20, 20, attention_mask=am)
    ref = mu.sdpa_mask(3, 20, 20, attention_mask=am.bool())
    assert full.dtype == torch.bool and torch.equal(full, ref)
    assert torch.equal(key_visible_of(full), am.bool())
    # causal & key padding is exactly the full mask: the factorisation the kernel relies on
    causal = torch.tril(torch.ones(20, 20, dtype=torch.bool))
    assert torch.equal(full, causal[None, None] & am.bool()[:, None, None, :])
    # cached decoding: one query against 20 keys (the diagonal offset is sk - sq)
    step = fused_attention_mask(3, 1, 20, q_offset=19, attention_mask=am)
    assert step is None or torch.equal(key_visible_of(step), am.bool())
    # another pattern (sliding window) carries no key part
    sw = fused_attention_mask(3, 20, 20, mask_function=mu.sliding_window_causal_mask_function(4), attention_mask=am)
    assert key_visible_of(sw) is None
    # a diagonal that is not the kernel's (queries offset against the keys) carries none either
    off = fused_attention_mask(3, 10, 20, q_offset=5, attention_mask=am)
    assert off is None or key_visible_of(off) is None
    # the pair survives a move or a no-op .to(), but no other operation, and a mask that was
    # written to in place after it was built no longer counts
    assert torch.equal(key_visible_of(full.to(full.device)), am.bool())
    assert torch.equal(key_visible_of(full.to("cpu", copy=True)), am.bool())
    assert key_visible_of(full[..., :20]) is None and key_visible_of(full.clone()) is None
    assert key_visible_of(full & full) is None and key_visible_of(full.to(torch.uint8)) is None
    edited = fused_attention_mask(3, 20, 20, attention_mask=am)
    edited[0, 0, 5, 2] = False  # e.g. a wrapper that cuts a window into the mask
    assert key_visible_of(edited) is None and isinstance(edited, torch.Tensor)


@pytest.mark.gpu
def test_causal_model_on_a_padded_batch_takes_the_causal_masked_kernel(device, monkeypatch):
    from oslo_amd.torch.nn.modules import functional as onn_f

    calls = []
    real = onn_f.scaled_masked_softmax_dropout

    def spy(input, mask, scale=1.0, p=0.0, training=True, causal=False):
        calls.append((tuple(mask.shape), causal))
        return real(input, mask, scale, p, training, causal=causal)

    monkeypatch.setattr(onn_f, "scaled_masked_softmax_dropout", spy)
    m = tiny_gpt2().to(device).eval()
    ids, am = inputs()
    ids, am = ids.to(device), am.to(device)
    with torch.no_grad():
        ref = m(ids, attention_mask=am).logits
    fused_scale_mask_softmax(m)
    with torch.no_grad():
        out = m(ids, attention_mask=am).logits
    valid = am.bool()
    assert (out[valid] - ref[valid]).abs().max().item() <= 2e-4
    b, s = ids.shape
    assert calls and all(shape == (b, 1, 1, s) and causal for shape, causal in calls), calls


@pytest.mark.gpu
def test_mask_moved_or_edited_between_builder_and_attention(device, monkeypatch):
    """The mask builder's result moved to the GPU still reaches the
    causal + key-padding kernel; the same mask written to in place afterwards
    (a window cut into it) is applied as it then is, by the kernel that reads
    the whole mask."""
    from oslo_amd.transformers.kernel_fusion_utils import (
        fused_attention_forward, fused_attention_mask)

    calls = _spy(monkeypatch, "scaled_masked_softmax_dropout")
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(3, 4, 20, 16, generator=g).to(device) for _ in range(3))
    am = torch.ones(3, 20, dtype=torch.long)
    am[1, 15:] = 0
    mask = fused_attention_mask(3, 20, 20, attention_mask=am)  # built on the CPU
    moved = mask.to(device)
    out, _ = fused_attention_forward(_AttnStub(True).eval(), q, k, v, moved, scaling=0.25)
    assert calls[-1][1].get("causal") is True and tuple(calls[-1][0][1].shape) == (3, 1, 1, 20)
    ref = _eager_attention(q, k, v, 0.25, torch.where(mask, 0.0, -10000.0).to(device))
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    moved[:, :, :, 0] = False          # in place: hide key 0 from every query but keep ...
    moved[:, :, 0, 0] = True           # ... query 0's only key
    out, _ = fused_attention_forward(_AttnStub(True).eval(), q, k, v, moved, scaling=0.25)
    assert not calls[-1][1].get("causal") and tuple(calls[-1][0][1].shape) == (3, 1, 20, 20)
    ref = _eager_attention(q, k, v, 0.25, torch.where(moved, 0.0, -10000.0))
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["gpt2", "bert"])
def test_fully_swapped_model_under_autocast_with_fp32_parameters(device, family):
    """torch.autocast with fp32 parameters: the GEMM outputs arrive in bf16, the
    biases and norm parameters are fp32.  The reference's TorchScript bodies
    take that through torch's promotion; the fused functions cast their
    operands to the autocast dtype, as the norm wrappers do.  Forward and
    backward of the fully swapped model against the unfused model under the
    same autocast."""
    from oslo_amd.transformers import fuse_all

    ids, am = inputs(b=3, s=32)
    ids, am = ids.to(device), am.to(device)
    if family == "gpt2":
        kw = dict(attn_pdrop=0.0, resid_pdrop=0.0, embd_pdrop=0.0)
        ref, fused = tiny_gpt2(seed=5, **kw).to(device).train(), tiny_gpt2(seed=5, **kw).to(device).train()
    else:
        # (the tanh form of GeLU, so that the intermediate blocks take the bias-GeLU kernel)
        kw = dict(hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, hidden_act="gelu_new")
        ref, fused = tiny_bert(seed=5, **kw).to(device).train(), tiny_bert(seed=5, **kw).to(device).train()
    changed = fuse_all(fused)
    assert changed["fused_bias_gelu"] > 0 and changed["fused_layer_norm"] + changed["fused_pre_ln_block"] > 0

    wproj = torch.randn(3, 32, 128, generator=torch.Generator().manual_seed(9)).to(device)

    def loss_of(m):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            if family == "gpt2":
                return m(ids, attention_mask=am, labels=ids).loss
            h = m(ids, attention_mask=am).last_hidden_state
            return (h.float() * wproj)[am.bool()].sum() / 64.0

    lr, lf = loss_of(ref), loss_of(fused)
    assert torch.isfinite(lf) and abs(lr.item() - lf.item()) <= 3e-2 * (abs(lr.item()) + 1.0)
    lr.backward()
    lf.backward()
    for (n, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        if pr.grad is None:
            continue
        assert pf.grad is not None and pf.grad.dtype == pr.grad.dtype == torch.float32, n
        # bf16 activations on both sides, rounded at different points (and the
        # unfused norms run in fp32 under autocast): compare in the L2 sense
        err = (pr.grad - pf.grad).norm().item()
        # (the absolute floor covers gradients that are zero in exact arithmetic,
        #  such as the key bias of an attention layer)
        assert err <= 0.1 * pr.grad.norm().item() + 1e-4, (n, err, pr.grad.norm().item())


@pytest.mark.gpu
def test_elementwise_functions_accept_what_torch_promotion_accepts(device):
    """bias / residual of another dtype follow x; a bias that is not a vector
    over the last dimension takes the torch formula."""
    x = torch.randn(6, 32, device=device, dtype=torch.bfloat16)
    b32 = torch.randn(32, device=device) * 0.1
    y = onn.fused_bias_gelu(x, b32)
    ref = onn.fused_bias_gelu(x, b32.to(torch.bfloat16))
    assert y.dtype == torch.bfloat16 and torch.equal(y, ref)
    r32 = torch.randn(6, 32, device=device)
    z = onn.fused_bias_dropout_add(x, b32, r32, 0.0, True)
    assert z.dtype == torch.bfloat16
    assert torch.equal(z, onn.fused_bias_dropout_add(x, b32.to(torch.bfloat16), r32.to(torch.bfloat16), 0.0, True))
    bcol = torch.randn(6, 1, device=device, dtype=torch.bfloat16)   # broadcasts over the columns
    w = onn.fused_bias_gelu(x, bcol)
    u = (x + bcol).float()
    want = u * 0.5 * (1.0 + torch.tanh(0.79788456 * u * (1 + 0.044715 * u * u)))
    assert (w.float() - want).abs().max().item() <= 3e-2
    with torch.autocast("cuda", dtype=torch.bfloat16):
        x32 = torch.randn(6, 32, device=device, requires_grad=True)
        b = torch.nn.Parameter(b32.clone())
        out = onn.fused_bias_gelu(x32, b)
        assert out.dtype == torch.bfloat16
        out.float().sum().backward()
    assert x32.grad.dtype == torch.float32 and b.grad.dtype == torch.float32 and b.grad.shape == (32,)
