"""``linear_cross_entropy``: fused lm-head linear + per-token log-prob + entropy with autograd.

Call-compatible with the reference's ``verl/utils/kernel/linear_cross_entropy.py:38-119``:
``linear_cross_entropy(hidden, weight, labels, temperature=1.0, reduction="none", dist_process_group=None)
-> (logprobs, entropy)``; outputs are fp32 and flattened to ``[T]`` (``logprobs`` is 0-dim for
``"sum"`` / ``"mean"``), ``d_hidden`` is viewed back to ``hidden``'s shape, ``d_weight`` has
``hidden.dtype``, the four non-tensor arguments get ``None`` gradients.  ``[T, V]`` logits are never
written to memory.
"""

from __future__ import annotations

import typing

import torch


class LinearCrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        hidden: torch.Tensor,
        weight: torch.Tensor,
        labels: torch.Tensor,
        temperature: typing.Optional[float] = 1.0,
        reduction: typing.Optional[str] = "none",
        dist_process_group=None,
    ):
        assert isinstance(temperature, float), f"temperature must be a float, but got {type(temperature)}"
        assert isinstance(reduction, str), f"reduction must be a str, but got {type(reduction)}"
        with torch.cuda.nvtx.range("LinearCrossEntropy-forward"):
            from . import kernels

            REDUCTION = kernels.get_entropy_reduction_enum_number(reduction.lower())
            original_hidden_shape = hidden.shape
            if len(hidden.shape) != 2:
                hidden = hidden.view(-1, hidden.shape[-1])
            if len(labels.shape) != 1:
                labels = labels.view(-1)
            logprobs, entropy, _maximum, _accumulate, _entropy_b = kernels.efficient_entropy_forward(
                hidden, weight, labels, REDUCTION, temperature, dist_process_group
            )
            ctx.save_for_backward(hidden, weight, labels, _maximum, _accumulate, _entropy_b)
            ctx.original_hidden_shape = original_hidden_shape
            ctx.REDUCTION = REDUCTION
            ctx.dist_process_group = dist_process_group
            ctx.should_return_fp32_grad = False
            ctx.temperature = temperature
            ctx.set_materialize_grads(False)  # an unused output arrives as None and costs nothing
        return logprobs, entropy

    @staticmethod
    def backward(ctx, dlogprobs: typing.Optional[torch.Tensor], dentropy: typing.Optional[torch.Tensor]):
        from . import kernels

        with torch.cuda.nvtx.range("LinearCrossEntropy-backward"):
            (hidden, weight, labels, _maximum, _accumulate, _entropy_b) = ctx.saved_tensors
            if dlogprobs is None:
                shape = (hidden.shape[0],) if ctx.REDUCTION == 0 else ()
                dlogprobs = torch.zeros(shape, device=hidden.device, dtype=torch.float32)
            d_hidden, d_weight = kernels.efficient_entropy_backward(
                dlogprobs,
                dentropy,
                hidden,
                weight,
                labels,
                _maximum,
                _accumulate,
                _entropy_b,
                ctx.REDUCTION,
                ctx.should_return_fp32_grad,
                ctx.temperature,
                ctx.dist_process_group,
            )
            d_hidden = d_hidden.view(ctx.original_hidden_shape)
        return (d_hidden, d_weight, None, None, None, None)


linear_cross_entropy = LinearCrossEntropy.apply
