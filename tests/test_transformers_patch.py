"""Patch layer for Hugging Face causal LMs (reference: cut_cross_entropy/transformers/*).

The reference ships no test of its own for this layer; the checks here are against the unpatched
model of the installed library: with labels, the patched forward must return the same loss (and the
same gradients) as the library's logits + cross-entropy path, without forming logits.
Tiny random-initialised configurations only -- nothing is downloaded.
"""

import pytest
import torch

transformers = pytest.importorskip("transformers")

from cut_cross_entropy.transformers import cce_patch  # noqa: E402
from cut_cross_entropy.transformers.patch import PATCH_TARGETS, cce_forward  # noqa: E402
from cut_cross_entropy.transformers.utils import PatchOptions  # noqa: E402


def _tiny(model_type, **extra):
    common = dict(
        vocab_size=1000,
        hidden_size=128,
        intermediate_size=256,
        num_hidden_layers=2,
        num_attention_heads=4,
        num_key_value_heads=2,
        max_position_embeddings=128,
        attn_implementation="eager",
    )
    common.update(extra)
    if model_type == "llama":
        return transformers.LlamaConfig(**common)
    if model_type == "gemma2":
        return transformers.Gemma2Config(head_dim=32, sliding_window=64, **common)
    if model_type == "qwen2":
        return transformers.Qwen2Config(**common)
    if model_type == "mistral":
        return transformers.MistralConfig(**common)
    raise ValueError(model_type)


def test_patch_options_use_lce():
    opts = PatchOptions("cce", "mean", "auto", False, False, True, True, train_only=True)
    labels = torch.zeros(2, 4, dtype=torch.long)
    assert not opts.use_lce(None, training=True)
    assert opts.use_lce(labels, training=True)
    assert not opts.use_lce(labels, training=False)
    opts.train_only = False
    assert opts.use_lce(labels, training=False)
    assert set(opts.to_kwargs()) == {
        "impl", "reduction", "filter_eps", "accum_e_fp32", "accum_c_fp32", "filter_e_grad", "filter_c_grad"}


def test_unknown_impl_and_model_type():
    with pytest.raises(ValueError):
        cce_patch("llama", impl="no_such_impl")
    with pytest.raises(RuntimeError):
        cce_patch("no_such_model_family")
    assert {"llama", "phi3", "gemma2", "mistral", "qwen2"} == set(PATCH_TARGETS)


def test_instance_patch_replaces_forward_only_there():
    cfg = _tiny("llama")
    model = transformers.LlamaForCausalLM(cfg)
    other = transformers.LlamaForCausalLM(cfg)
    patched = cce_patch(model, impl="cce")
    assert patched is model
    assert model.forward.__func__ is cce_forward
    assert other.forward.__func__ is not cce_forward
    # without labels the patched forward is the ordinary logits path (runs on the CPU)
    ids = torch.randint(0, cfg.vocab_size, (2, 8))
    with torch.no_grad():
        a = model(input_ids=ids).logits
        b = transformers.LlamaForCausalLM.forward(model, input_ids=ids).logits
    assert torch.equal(a, b)


def test_instance_of_wrong_family_is_rejected():
    model = transformers.LlamaForCausalLM(_tiny("llama"))
    model.config.model_type = "qwen2"
    with pytest.raises(AssertionError):
        cce_patch(model)


@pytest.mark.gpu
@pytest.mark.parametrize("model_type", ["llama", "gemma2", "qwen2", "mistral"])
@pytest.mark.parametrize("impl", ["cce", "cce_exact"])
def test_patched_loss_and_grads_match_library(model_type, impl):
    torch.manual_seed(0)
    extra = {"final_logit_softcapping": 30.0} if model_type == "gemma2" else {}
    cfg = _tiny(model_type, **extra)
    cls = {"llama": transformers.LlamaForCausalLM, "gemma2": transformers.Gemma2ForCausalLM,
           "qwen2": transformers.Qwen2ForCausalLM, "mistral": transformers.MistralForCausalLM}[model_type]
    model = cls(cfg).to(device="cuda", dtype=torch.bfloat16)
    model.train()
    ids = torch.randint(0, cfg.vocab_size, (4, 64), device="cuda")
    labels = ids.clone()
    labels[:, :5] = -100

    ref = model(input_ids=ids, labels=labels)
    ref.loss.backward()
    ref_head = model.lm_head.weight.grad.float().clone()
    ref_embed_norm = model.model.layers[0].mlp.down_proj.weight.grad.float().clone()
    model.zero_grad(set_to_none=True)

    cce_patch(model, impl=impl)
    out = model(input_ids=ids, labels=labels)
    assert out.logits is None
    out.loss.backward()
    head = model.lm_head.weight.grad.float()
    inner = model.model.layers[0].mlp.down_proj.weight.grad.float()

    # the library rounds its logits to bf16 before the loss; the fused path never does: 1e-2 is that rounding
    assert abs(out.loss.item() - ref.loss.item()) <= 1e-2 * max(1.0, abs(ref.loss.item()))
    assert torch.allclose(head, ref_head, atol=2e-3, rtol=5e-2), (head - ref_head).abs().max()
    assert torch.allclose(inner, ref_embed_norm, atol=2e-3, rtol=5e-2), (inner - ref_embed_norm).abs().max()


@pytest.mark.gpu
def test_num_items_in_batch_turns_mean_into_scaled_sum():
    torch.manual_seed(0)
    cfg = _tiny("llama")
    model = transformers.LlamaForCausalLM(cfg).to(device="cuda", dtype=torch.bfloat16)
    ids = torch.randint(0, cfg.vocab_size, (2, 32), device="cuda")
    cce_patch(model, impl="cce")
    mean = model(input_ids=ids, labels=ids).loss
    n_valid = ids[:, 1:].numel()
    scaled = model(input_ids=ids, labels=ids, num_items_in_batch=2 * n_valid).loss
    assert abs(scaled.item() - 0.5 * mean.item()) <= 1e-3 * abs(mean.item())


@pytest.mark.gpu
def test_family_patch_applies_to_new_instances():
    from transformers.models.mistral import modeling_mistral

    original = modeling_mistral.MistralForCausalLM.forward
    try:
        assert cce_patch("mistral", impl="cce", train_only=True) is None
        torch.manual_seed(0)
        cfg = _tiny("mistral")
        model = transformers.MistralForCausalLM(cfg).to(device="cuda", dtype=torch.bfloat16)
        ids = torch.randint(0, cfg.vocab_size, (2, 32), device="cuda")
        model.train()
        assert model(input_ids=ids, labels=ids).logits is None
        model.eval()  # train_only: eval mode takes the library's own path
        assert model(input_ids=ids, labels=ids).logits is not None
    finally:
        modeling_mistral.MistralForCausalLM.forward = original
        if hasattr(modeling_mistral.MistralForCausalLM, "_cce_patch_options"):
            delattr(modeling_mistral.MistralForCausalLM, "_cce_patch_options")
