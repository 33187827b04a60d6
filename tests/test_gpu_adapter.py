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
