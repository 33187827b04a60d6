"""Adapter routing on the CPU with the kernel patched out, mirroring the reference's
tests/models/test_fused_kernels_ulysses_sp_on_cpu.py:156-290: ``shift_labels`` must be used verbatim,
otherwise labels / input_ids are rolled by one; the adapter must hand hidden states and the lm-head
weight to ``linear_cross_entropy`` and return its outputs untouched."""

import types

import pytest
import torch

from verl_amd.models.transformers import dense_common, monkey_patch


class _Model(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.config = types.SimpleNamespace(output_attentions=False, output_hidden_states=False, model_type="llama")
        self.lm_head = torch.nn.Linear(4, 9, bias=False)
        self._h = None

    def model(self, input_ids=None, **kw):
        h = torch.arange(input_ids.numel() * 4, dtype=torch.float32).view(*input_ids.shape, 4)

        class Out(tuple):
            past_key_values = None
            hidden_states = None
            attentions = None

        return Out((h,))


@pytest.fixture
def captured(monkeypatch):
    calls = {}

    def fake(hidden, weight, labels, temperature, reduction):
        calls.update(hidden=hidden, weight=weight, labels=labels, temperature=temperature, reduction=reduction)
        return torch.zeros(labels.numel()), torch.ones(labels.numel())

    monkeypatch.setattr(dense_common, "linear_cross_entropy", fake)
    from verl_amd.utils.experimental import torch_functional as experimental

    monkeypatch.setattr(experimental, "linear_cross_entropy", fake)
    return calls


def test_shift_labels_used_verbatim_else_rolled(captured):
    m = _Model()
    ids = torch.tensor([[5, 6, 7, 8]])
    out = dense_common.forward_with_hip_backend(m, input_ids=ids, return_dict=True, temperature=0.7)
    assert captured["labels"].tolist() == [[6, 7, 8, 5]] and captured["temperature"] == 0.7
    assert captured["reduction"] == "none" and captured["weight"] is not None
    assert out.log_probs.shape == (4,) and out.entropy.sum() == 4
    dense_common.forward_with_hip_backend(m, input_ids=ids, labels=torch.tensor([[1, 2, 3, 4]]), return_dict=True)
    assert captured["labels"].tolist() == [[2, 3, 4, 1]]
    sl = torch.tensor([[9, 9, 9, 9]])
    dense_common.forward_with_hip_backend(m, input_ids=ids, shift_labels=sl, return_dict=True)
    assert captured["labels"].tolist() == [[9, 9, 9, 9]]
    with pytest.raises(NotImplementedError):
        dense_common.forward_with_hip_backend(m, input_ids=ids, return_dict=False)


def test_patch_selection(captured, capsys):
    class M(_Model):
        pass

    m = M()
    orig = M.forward
    monkey_patch.patch_forward_with_backends(m, use_fused_kernels=False, fused_kernels_backend="hip")
    assert M.forward is orig
    monkey_patch.patch_forward_with_backends(m, use_fused_kernels=True, fused_kernels_backend="bogus")
    assert M.forward is orig
    # the reference installs its triton forward for "triton" and its torch forward for "torch" / "liger"
    # (verl/models/transformers/monkey_patch.py:281-291); the two differ in the shape and dtype of what they return
    for backend, fwd in (("triton", dense_common.forward_with_hip_backend), ("hip", dense_common.forward_with_hip_backend),
                         ("torch", dense_common.forward_with_torch_backend), ("liger", dense_common.forward_with_torch_backend)):
        monkey_patch.patch_forward_with_backends(m, use_fused_kernels=True, fused_kernels_backend=backend)
        assert M.forward is fwd and m._verl_fused_kernels_backend == backend
    m.config.model_type = "qwen2_vl"
    with pytest.raises(NotImplementedError):
        monkey_patch.patch_forward_with_backends(m, use_fused_kernels=True, fused_kernels_backend="hip")


def test_torch_backend_returns_batch_shaped_outputs(captured):
    """forward_with_torch_backend goes through FusedLinearForPPO (verl/models/transformers/dense_common.py:119-129):
    outputs shaped like input_ids, entropy in the hidden dtype, so that output.log_probs[:, -R-1:-1] slices responses."""
    m = _Model()
    m._verl_fused_kernels_backend = "torch"
    ids = torch.tensor([[5, 6, 7, 8], [1, 2, 3, 4]])
    out = dense_common.forward_with_torch_backend(m, input_ids=ids, return_dict=True, temperature=0.5)
    assert out.log_probs.shape == (2, 4) and out.entropy.shape == (2, 4) and out.entropy.dtype == torch.float32
    assert captured["labels"].tolist() == [6, 7, 8, 5, 2, 3, 4, 1] and captured["temperature"] == 0.5
    assert out.log_probs[:, -3:-1].shape == (2, 2)
