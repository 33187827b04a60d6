"""``linear_cross_entropy``: fused lm-head linear + per-token log-prob + entropy with autograd.

Call-compatible with the reference's ``verl/utils/kernel/linear_cross_entropy.py:38-119``:
``linear_cross_entropy(hidden, weight, labels, temperature=1.0, reduction="none", dist_process_group=None)
-> (logprobs, entropy)``; outputs are fp32 and flattened to ``[T]`` (``logprobs`` is 0-dim for
``"sum"`` / ``"mean"``), ``d_hidden`` comes back in ``hidden``'s shape, ``d_weight`` has ``hidden.dtype``, the four
non-tensor arguments get ``None`` gradients.  ``[T, V]`` logits are never written to memory, except while they are no
larger than the weight (at most half the hidden size in tokens), where the node keeps them in fp32 for
its backward (it saves the backward the pass over ``[V, H]`` and the product that recompute them).

The autograd node is a thin shell: everything it does besides argument checks and reshapes happens in the two host
launchers of ``kernels.py`` (one C-ABI call each).
"""

from __future__ import annotations

import threading
import typing
import weakref

import torch

from ... import _abi
from . import kernels


def _as_token_rows(hidden: torch.Tensor, labels: torch.Tensor):
    """``[..., H]`` / ``[...]`` viewed as ``[T, H]`` / ``[T]`` (views, like the reference: a tensor that cannot be
    viewed raises)."""
    rows = hidden if hidden.dim() == 2 else hidden.view(-1, hidden.shape[-1])
    flat = labels if labels.dim() == 1 else labels.view(-1)
    return rows, flat


class LinearCrossEntropy(torch.autograd.Function):
    """``apply(hidden, weight, labels, temperature, reduction, dist_process_group)``."""

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
        # the reference's two type checks (:64-65), messages included: callers' tests match on them
        assert isinstance(temperature, float), f"temperature must be a float, but got {type(temperature)}"
        assert isinstance(reduction, str), f"reduction must be a str, but got {type(reduction)}"
        # the reference's profiler range (:66); on ROCm torch.cuda.nvtx is roctx, so `rocprofv3 --marker-trace` shows it
        torch.cuda.nvtx.range_push("LinearCrossEntropy-forward")
        try:
            mode = kernels.get_entropy_reduction_enum_number(reduction.lower())
            rows, flat_labels = _as_token_rows(hidden, labels)
            # (no backward will follow, under no_grad or with inputs that take no gradient: nothing is kept beyond the outputs;
            # nor when the logits that earlier calls keep, together with this call's, would pass what ONE call may keep)
            keep = getattr(_caller, "grad_enabled", True) and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
            keep = keep and _room_for_logits(rows, weight)
            logprobs, entropy, *stats, cache = kernels.forward_keeping_logits(
                rows, weight, flat_labels, mode, temperature, dist_process_group, keep_logits=keep
            )
            if cache is not None:
                _account(cache)
            # stats = (maximum, accumulate, entropy_b), fp32 [T]; cache: the logits, with few tokens only (else None)
            ctx.save_for_backward(rows, weight, flat_labels, *stats, cache)
            ctx.call = (hidden.shape, mode, temperature, dist_process_group)
            ctx.set_materialize_grads(False)  # an unused output arrives as None and costs nothing
        finally:
            torch.cuda.nvtx.range_pop()
        return logprobs, entropy

    @staticmethod
    def backward(ctx, dlogprobs: typing.Optional[torch.Tensor], dentropy: typing.Optional[torch.Tensor]):
        torch.cuda.nvtx.range_push("LinearCrossEntropy-backward")  # the reference's range (:93)
        try:
            rows, weight, flat_labels, maximum, accumulate, entropy_b, cache = ctx.saved_tensors
            shape, mode, temperature, group = ctx.call
            if dlogprobs is None:  # only the entropy was used downstream
                dlogprobs = torch.zeros((rows.shape[0],) if mode == 0 else (), device=rows.device, dtype=torch.float32)
            # a gradient that autograd does not ask for (a frozen lm-head under LoRA, detached hidden states) is not computed
            need_hidden, need_weight = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
            d_rows, d_weight = kernels.efficient_entropy_backward(
                dlogprobs, dentropy, rows, weight, flat_labels, maximum, accumulate, entropy_b, mode,
                False,  # should_return_fp32_grad: autograd wants the inputs' dtype
                temperature, group, need_d_hidden=need_hidden, need_d_weight=need_weight, logits_cache=cache,
            )  # fmt: skip
        finally:
            torch.cuda.nvtx.range_pop()
        return (d_rows.view(shape) if d_rows is not None else None), d_weight, None, None, None, None


# what torch.is_grad_enabled() said where linear_cross_entropy was called (inside Function.forward it is always off)
_caller = threading.local()

# Kept logits are bounded per device IN AGGREGATE, not only per call: a caller that cuts a long batch into pieces of a
# few hundred tokens inside one autograd graph (to bound memory, as the reference's chunked torch backend does) would
# otherwise end up holding fp32 logits for the whole batch.  Bytes of logits alive per device index:
_kept_bytes: dict[int, int] = {}
_kept_lock = threading.Lock()


def kept_logits_bytes(device=None) -> int:
    """Bytes of kept logits that autograd graphs on ``device`` (default: the current one) hold right now."""
    index = torch.device("cuda", torch.cuda.current_device()).index if device is None else torch.device(device).index
    return _kept_bytes.get(index, 0)


def _row_bytes(weight: torch.Tensor) -> int:
    return (weight.shape[0] + 63) // 64 * 64 * 4


def _room_for_logits(rows: torch.Tensor, weight: torch.Tensor) -> bool:
    """All live caches of a device together stay within what ONE call may keep at most for this weight."""
    if not (rows.is_cuda and weight.dim() == 2 and weight.dtype in (torch.bfloat16, torch.float16)):
        return False  # (nothing is kept for fp32; anything else is the launcher's to refuse)
    most = _abi.load().lce_logits_cache_max_tokens(weight.shape[1], _abi.dtype_code(weight.dtype))
    want = rows.shape[0] * _row_bytes(weight)
    return _kept_bytes.get(rows.device.index, 0) + want <= most * _row_bytes(weight)


def _release(index: int, nbytes: int) -> None:
    with _kept_lock:
        _kept_bytes[index] = _kept_bytes.get(index, 0) - nbytes


def _account(cache: torch.Tensor) -> None:
    nbytes = cache.numel() * cache.element_size()
    with _kept_lock:
        _kept_bytes[cache.device.index] = _kept_bytes.get(cache.device.index, 0) + nbytes
    weakref.finalize(cache, _release, cache.device.index, nbytes)  # when the graph that saved it lets go of it


def linear_cross_entropy(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: typing.Optional[float] = 1.0,
    reduction: typing.Optional[str] = "none",
    dist_process_group=None,
):
    """``LinearCrossEntropy.apply`` with the reference's argument list (the reference binds the name to ``apply`` itself,
    verl/utils/kernel/linear_cross_entropy.py:119)."""
    _caller.grad_enabled = torch.is_grad_enabled()
    try:
        return LinearCrossEntropy.apply(hidden, weight, labels, temperature, reduction, dist_process_group)
    finally:
        _caller.grad_enabled = True
