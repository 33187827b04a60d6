"""``FusedLinearForPPO``: module-style front end of the fused lm-head log-prob + entropy.

Mirrors the reference's ``verl/utils/experimental/torch_functional.py:220-269``: constructor
``(chunk_size=512, impl_backend="torch")``, ``forward(hidden_states, vocab_weights, input_ids,
temperature=1.0) -> (log_probs, entropy)`` shaped like ``input_ids``; unlike
``linear_cross_entropy`` the outputs are reshaped back and the entropy carries the input dtype
(:58, :143-145).  Every backend name the reference accepts ("torch", "liger") is served by the same
HIP kernels here; ``chunk_size`` is accepted and unused (nothing ``[chunk, V]`` is materialised).

The reference's torch backend takes any hidden size (its sequence-parallel test runs ``hidden_size=64``,
tests/special_distributed/test_fused_kernels_ulysses_sp.py:47-60), while the MFMA kernels want whole
128-element K slabs: a hidden size that is not a multiple of 128 is zero-padded up to one on both operands
(zero columns add nothing to any logit, and autograd drops their gradient columns again).  That costs a copy
of the weight per call and is meant for tests and toy models; production heads are multiples of 128.
"""

from __future__ import annotations

import torch

from ..kernel.linear_cross_entropy import linear_cross_entropy


class FusedLinearForPPO(torch.nn.Module):
    def __init__(self, chunk_size: int = 512, impl_backend: str = "torch"):
        super().__init__()
        if impl_backend not in ("torch", "liger", "hip"):
            raise ValueError(f"Unsupported FusedLinearForPPO backend: {impl_backend}. Choose 'torch', 'liger' or 'hip'.")
        self.chunk_size = chunk_size
        self.impl_backend = impl_backend

    def forward(self, hidden_states, vocab_weights, input_ids, temperature: float = 1.0):
        input_ids = input_ids.to(torch.int64)
        if hidden_states.dim() not in (2, 3):
            raise ValueError(f"hidden_states must be 2-D or 3-D, got {hidden_states.dim()}-D")
        if hidden_states.shape[:-1] != input_ids.shape:
            raise ValueError("hidden_states and input_ids disagree on the token dimensions")
        h2 = hidden_states.reshape(-1, hidden_states.shape[-1])
        if not h2.is_contiguous():
            h2 = h2.contiguous()
        w = vocab_weights if vocab_weights.is_contiguous() else vocab_weights.contiguous()
        pad = -h2.shape[-1] % 128
        if pad:
            h2 = torch.nn.functional.pad(h2, (0, pad))
            w = torch.nn.functional.pad(w, (0, pad))
        log_probs, entropy = linear_cross_entropy(h2, w, input_ids.reshape(-1), float(temperature), "none")
        return log_probs.view(input_ids.shape), entropy.view(input_ids.shape).to(hidden_states.dtype)
