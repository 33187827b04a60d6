"""End to end through a real (tiny, offline-built) HF model, like the reference's
tests/special_distributed/test_fused_kernels_ulysses_sp.py:47-60: the patched forward's log-probs and
entropy must match the unfused route (model logits -> oracle)."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu


def test_patched_llama_matches_unfused_logits():
    from transformers import AutoModelForCausalLM, LlamaConfig

    from verl_amd.models.transformers.monkey_patch import patch_forward_with_backends

    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=1000, hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128)
    model = AutoModelForCausalLM.from_config(cfg).to("cuda:0", torch.bfloat16)
    ids = torch.randint(0, 1000, (2, 37), device="cuda:0")
    with torch.no_grad():
        logits = model(input_ids=ids).logits  # [2, 37, V] bf16
        hidden = model.model(input_ids=ids)[0]
    labels = torch.roll(ids, -1, -1)
    want_lp, want_ent = O.lce_forward(hidden, model.lm_head.weight, labels, 0.9)
    patch_forward_with_backends(model, use_fused_kernels=True, fused_kernels_backend="triton")
    out = model(input_ids=ids, temperature=0.9, return_dict=True)
    assert out.log_probs.shape == (2 * 37,) and out.logits is None
    torch.testing.assert_close(out.log_probs, want_lp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(out.entropy, want_ent, atol=5e-3, rtol=5e-4)
    # and against the bf16 logits the unfused model produced (coarser: those logits were rounded to bf16)
    ref_lp = O.logprobs_from_logits(logits.float() / 0.9, labels).reshape(-1)
    torch.testing.assert_close(out.log_probs, ref_lp, atol=5e-2, rtol=2e-2)
    # gradients flow into the model through the fused head
    out.log_probs.sum().backward()
    assert model.lm_head.weight.grad is not None and torch.isfinite(model.lm_head.weight.grad).all()
    assert model.model.embed_tokens.weight.grad.abs().sum() > 0


@pytest.mark.parametrize("backend", ["triton", "hip", "torch", "liger"])
def test_output_shape_and_dtype_per_backend_name(backend):
    """Every backend name verl's configuration can carry gives what that backend gives in the reference
    (verl/models/transformers/dense_common.py:119-129 against :189-195): flat fp32 vectors for triton, [batch, seq]
    with the entropy in the hidden dtype for torch / liger (the padded engines slice log_probs[:, -R-1:-1])."""
    from transformers import AutoModelForCausalLM, LlamaConfig

    from verl_amd.models.transformers.monkey_patch import patch_forward_with_backends

    torch.manual_seed(1)
    cfg = LlamaConfig(vocab_size=512, hidden_size=128, intermediate_size=256, num_hidden_layers=1,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=64)
    model = AutoModelForCausalLM.from_config(cfg).to("cuda:0", torch.bfloat16)
    B, S = 3, 21
    ids = torch.randint(0, 512, (B, S), device="cuda:0")
    with torch.no_grad():
        hidden = model.model(input_ids=ids)[0]
    want_lp, want_ent = O.lce_forward(hidden, model.lm_head.weight, torch.roll(ids, -1, -1), 1.0)
    patch_forward_with_backends(model, use_fused_kernels=True, fused_kernels_backend=backend)
    with torch.no_grad():
        out = model(input_ids=ids, temperature=1.0, return_dict=True)
    if backend in ("triton", "hip"):
        assert out.log_probs.shape == (B * S,) and out.entropy.shape == (B * S,)
        assert out.log_probs.dtype == torch.float32 and out.entropy.dtype == torch.float32
    else:
        assert out.log_probs.shape == (B, S) and out.entropy.shape == (B, S)
        assert out.log_probs.dtype == torch.float32 and out.entropy.dtype == torch.bfloat16
        assert out.log_probs[:, -5 - 1 : -1].shape == (B, 5)
    torch.testing.assert_close(out.log_probs.reshape(-1), want_lp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(out.entropy.reshape(-1).float(), want_ent, atol=2e-2, rtol=1e-2)


def _tiny_text(**more):
    cfg = dict(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
               vocab_size=512, max_position_embeddings=256, bos_token_id=1, eos_token_id=2, pad_token_id=0)
    cfg.update(more)
    return cfg


_VISION = dict(depth=1, hidden_size=32, out_hidden_size=128, num_heads=2, intermediate_size=64)
_MROPE = {"rope_type": "default", "mrope_section": [4, 6, 6]}
_LINEAR = dict(head_dim=32, linear_num_key_heads=2, linear_num_value_heads=4, linear_key_head_dim=16, linear_value_head_dim=16,
               layer_types=["linear_attention", "full_attention"])
_MULTIMODAL = {
    # model_type: (config class, model class, config arguments)
    "qwen2_vl": ("Qwen2VLConfig", "Qwen2VLForConditionalGeneration",
                 dict(text_config=_tiny_text(rope_scaling={"type": "mrope", "mrope_section": [4, 6, 6]}),
                      vision_config=dict(depth=1, embed_dim=32, hidden_size=128, num_heads=2, mlp_ratio=2))),
    "qwen2_5_vl": ("Qwen2_5_VLConfig", "Qwen2_5_VLForConditionalGeneration",
                   dict(text_config=_tiny_text(rope_scaling={"type": "mrope", "mrope_section": [4, 6, 6]}),
                        vision_config=dict(_VISION, fullatt_block_indexes=[0]))),
    "glm4v": ("Glm4vConfig", "Glm4vForConditionalGeneration", dict(text_config=_tiny_text(rope_scaling=_MROPE), vision_config=_VISION)),
    "qwen3_vl": ("Qwen3VLConfig", "Qwen3VLForConditionalGeneration",
                 dict(text_config=_tiny_text(head_dim=32, rope_scaling=dict(_MROPE, mrope_interleaved=True)),
                      vision_config=dict(_VISION, deepstack_visual_indexes=[0]))),
    "qwen3_vl_moe": ("Qwen3VLMoeConfig", "Qwen3VLMoeForConditionalGeneration",
                     dict(text_config=_tiny_text(head_dim=32, moe_intermediate_size=64, num_experts=4, num_experts_per_tok=2,
                                                 rope_scaling=dict(_MROPE, mrope_interleaved=True)),
                          vision_config=dict(_VISION, deepstack_visual_indexes=[0]))),
    "qwen3_5": ("Qwen3_5Config", "Qwen3_5ForConditionalGeneration", dict(text_config=_tiny_text(**_LINEAR), vision_config=_VISION)),
    "qwen3_5_moe": ("Qwen3_5MoeConfig", "Qwen3_5MoeForConditionalGeneration",
                    dict(text_config=_tiny_text(moe_intermediate_size=64, shared_expert_intermediate_size=64, num_experts=4,
                                                num_experts_per_tok=2, **_LINEAR), vision_config=_VISION)),
}


@pytest.mark.parametrize("model_type", sorted(_MULTIMODAL))
def test_patched_multimodal_model_matches_its_unfused_logits(model_type):
    """The model types the reference patches with forwards of their own (verl/models/transformers/monkey_patch.py:255-274),
    built tiny and offline from their configs, text-only batch with the (4, batch, seq) position ids of verl's data
    pipeline: the patched forward's log-probs and entropy against the oracle on the model's own hidden states and
    against its unfused logits, for the flat and for the shaped backend; gradients reach the embeddings."""
    import transformers

    from verl_amd.models.transformers.monkey_patch import patch_forward_with_backends

    config_cls, model_cls, arguments = _MULTIMODAL[model_type]
    if not hasattr(transformers, model_cls):
        pytest.skip(f"transformers {transformers.__version__} has no {model_cls}")
    torch.manual_seed(3)
    config = getattr(transformers, config_cls)(**arguments)
    assert config.model_type == model_type
    model = getattr(transformers, model_cls)(config).to("cuda:0", torch.bfloat16)
    B, S, tau = 2, 24, 0.8
    ids = torch.randint(3, 512, (B, S), device="cuda:0")
    mask = torch.ones_like(ids)
    pos = torch.arange(S, device="cuda:0")[None, None].expand(4, B, S).contiguous()
    with torch.no_grad():
        unfused = model(input_ids=ids, attention_mask=mask, position_ids=pos)
        hidden = model.model(input_ids=ids, attention_mask=mask, position_ids=pos)[0]
    labels = torch.roll(ids, -1, -1)
    want_lp, want_ent = O.lce_forward(hidden, model.lm_head.weight, labels, tau)
    from_logits = O.logprobs_from_logits(unfused.logits.float() / tau, labels).reshape(-1)

    patch_forward_with_backends(model, use_fused_kernels=True, fused_kernels_backend="triton")
    out = model(input_ids=ids, attention_mask=mask, position_ids=pos, temperature=tau)
    assert type(out).__name__.endswith("CausalLMOutputForPPO") and out.logits is None
    assert out.log_probs.shape == (B * S,) and out.log_probs.dtype == torch.float32 and out.entropy.shape == (B * S,)
    torch.testing.assert_close(out.log_probs, want_lp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(out.entropy, want_ent, atol=5e-3, rtol=5e-4)
    torch.testing.assert_close(out.log_probs, from_logits, atol=5e-2, rtol=2e-2)  # (those logits were rounded to bf16)
    (out.log_probs.sum() + out.entropy.sum()).backward()
    embed = model.get_input_embeddings().weight
    assert torch.isfinite(model.lm_head.weight.grad).all() and embed.grad is not None and embed.grad.abs().sum() > 0

    patch_forward_with_backends(model, use_fused_kernels=True, fused_kernels_backend="torch")
    with torch.no_grad():
        shaped = model(input_ids=ids, attention_mask=mask, position_ids=pos, temperature=tau, shift_labels=labels)
    assert shaped.log_probs.shape == (B, S) and shaped.entropy.shape == (B, S) and shaped.entropy.dtype == torch.bfloat16
    torch.testing.assert_close(shaped.log_probs.reshape(-1), want_lp, atol=1e-3, rtol=2e-4)
    if model_type in ("qwen2_vl", "qwen2_5_vl", "glm4v"):
        with pytest.raises(ValueError, match="position_ids"):
            model(input_ids=ids, attention_mask=mask, position_ids=pos[1:], temperature=tau)
