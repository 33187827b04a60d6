"""``FusedLinearForPPO``: module-style front end of the fused lm-head log-prob + entropy.

Mirrors the reference's ``verl/utils/experimental/torch_functional.py:220-269``: constructor
``(chunk_size=512, impl_backend="torch")``, ``forward(hidden_states, vocab_weights, input_ids,
temperature=1.0) -> (log_probs, entropy)`` shaped like ``input_ids``; unlike
``linear_cross_entropy`` the outputs are reshaped back and the entropy carries the input dtype
(:58, :143-145).  Every backend name the reference accepts ("torch", "liger") is served by the same
HIP kernels here; ``chunk_size`` is accepted and unused (nothing ``[chunk, V]`` is materialised).
"""

from __future__ import annotations

import torch

from ..kernel.linear_cross_entropy import linear_cross_entropy


class FusedLinearForPPO(torch.nn.Module):
    def __init__(self, chunk_size: int = 512, impl_backend: str = "torch"):
        super().__init__()
        if impl_backend not in ("torch", "liger", "hip"):
            raise ValueError(f"Unsupported impl_backend: {impl_backend}")
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
        log_probs, entropy = linear_cross_entropy(h2, w, input_ids.reshape(-1), float(temperature), "none")
        return log_probs.view(input_ids.shape), entropy.view(input_ids.shape).to(hidden_states.dtype)
