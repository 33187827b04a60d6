"""Unfused twins on logits that already exist: ``logprobs_from_logits`` and ``entropy_from_logits``.

Same signatures and result dtypes/shapes as the reference's ``verl/utils/torch_functional.py``
(``gather_from_labels`` :50-70, ``logprobs_from_logits`` :73-107, ``logprobs_from_logits_flash_attn`` :110-133,
``logprobs_from_logits_naive`` :155-170,
``logprobs_from_logits_v2`` :173-207, ``entropy_from_logits`` :231-245, ``entropy_from_logits_with_chunking``
:248-270, ``masked_sum`` :273-291, ``masked_mean`` :294-308, ``calculate_sum_pi_squared_from_logits`` :687-703).  The row reductions run as single-pass
HIP kernels (one read of the logits; fp32 arithmetic whatever the storage dtype) with an autograd
backward that is one more fused pass; there is no eager fallback on this path.
"""

from __future__ import annotations

import torch

from .. import _abi


def gather_from_labels(data: torch.Tensor, label: torch.Tensor) -> torch.Tensor:
    return torch.gather(data, -1, label.unsqueeze(-1)).squeeze(-1)


def _as_rows(logits: torch.Tensor):
    V = logits.shape[-1]
    rows = logits.reshape(-1, V)
    if rows.stride(-1) != 1:
        rows = rows.contiguous()
    return rows, V


def _require_gpu(logits: torch.Tensor) -> None:
    """The reference's twins run on any device; these are HIP kernels and there is no eager fallback."""
    if not logits.is_cuda:
        raise _abi.LceError(
            "verl_amd.utils.torch_functional runs on GPU tensors only (hand-written HIP kernels, no CPU or eager "
            f"fallback); got a tensor on {logits.device}"
        )


def _logits_forward(logits, labels, want_logprobs: bool, want_entropy: bool, want_stats: bool):
    _require_gpu(logits)
    code = _abi.dtype_code(logits.dtype)
    rows, V = _as_rows(logits)
    R = rows.shape[0]
    dev = logits.device
    lp = torch.empty((R,), device=dev, dtype=torch.float32) if want_logprobs else None
    ent = torch.empty((R,), device=dev, dtype=torch.float32) if want_entropy else None
    # row statistics for the backward (it then needs one pass instead of two)
    # (the caller decides: inside autograd.Function.forward grad mode is off, so it cannot be read here)
    stats = torch.empty((R, 2), device=dev, dtype=torch.float32) if want_stats else None
    y = None
    if want_logprobs:
        y = labels.reshape(-1).to(torch.int64).contiguous()
        assert y.shape[0] == R and y.device == dev
    if R > 0:
        with torch.cuda.device(dev):
            rc = _abi.load().lce_logits_forward(
                rows.data_ptr(), rows.stride(0), _abi.ptr(y), R, V, code, _abi.ptr(lp), _abi.ptr(ent), _abi.ptr(stats),
                _abi.current_stream(dev),
            )  # fmt: skip
            _abi.check(rc, "lce_logits_forward")
    return rows, y, lp, ent, stats


def _logits_backward(rows, y, stats, g_lp, g_ent, out_shape, out_dtype):
    R, V = rows.shape
    dev = rows.device
    d = torch.empty((R, V), device=dev, dtype=rows.dtype)
    g_lp = None if g_lp is None else g_lp.reshape(-1).to(torch.float32).contiguous()
    g_ent = None if g_ent is None else g_ent.reshape(-1).to(torch.float32).contiguous()
    if R > 0:
        with torch.cuda.device(dev):
            rc = _abi.load().lce_logits_backward(
                rows.data_ptr(), rows.stride(0), _abi.ptr(y), R, V, _abi.dtype_code(rows.dtype), _abi.ptr(stats),
                _abi.ptr(g_lp), _abi.ptr(g_ent), d.data_ptr(), d.stride(0), _abi.current_stream(dev),
            )  # fmt: skip
            _abi.check(rc, "lce_logits_backward")
    return d.reshape(out_shape).to(out_dtype)


class _LogprobsFromLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels):
        rows, y, lp, _, stats = _logits_forward(logits, labels, True, False, ctx.needs_input_grad[0])
        ctx.save_for_backward(rows, y, stats)
        ctx.shape, ctx.dtype = logits.shape, logits.dtype
        return lp.reshape(logits.shape[:-1]).to(logits.dtype)

    @staticmethod
    def backward(ctx, g):
        rows, y, stats = ctx.saved_tensors
        return _logits_backward(rows, y, stats, g, None, ctx.shape, ctx.dtype), None


class _EntropyFromLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, out_dtype):
        rows, _, _, ent, stats = _logits_forward(logits, None, False, True, ctx.needs_input_grad[0])
        ctx.save_for_backward(rows, stats)
        ctx.shape, ctx.dtype = logits.shape, logits.dtype
        return ent.reshape(logits.shape[:-1]).to(out_dtype)

    @staticmethod
    def backward(ctx, g):
        rows, stats = ctx.saved_tensors
        return _logits_backward(rows, None, stats, None, g, ctx.shape, ctx.dtype), None


class _LogprobsAndEntropyFromLogits(torch.autograd.Function):
    """Both row reductions from one read of the logits, and ONE gradient of the logits in the backward."""

    @staticmethod
    def forward(ctx, logits, labels, entropy_dtype):
        rows, y, lp, ent, stats = _logits_forward(logits, labels, True, True, ctx.needs_input_grad[0])
        ctx.save_for_backward(rows, y, stats)
        ctx.shape, ctx.dtype = logits.shape, logits.dtype
        ctx.set_materialize_grads(False)
        return lp.reshape(logits.shape[:-1]).to(logits.dtype), ent.reshape(logits.shape[:-1]).to(entropy_dtype)

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        rows, y, stats = ctx.saved_tensors
        if g_lp is None and g_ent is None:
            return None, None, None
        return _logits_backward(rows, y if g_lp is not None else None, stats, g_lp, g_ent, ctx.shape, ctx.dtype), None, None


def logprobs_and_entropy_from_logits(logits, labels, entropy_dtype=None):
    """``(logprobs_from_logits(logits, labels), entropy_from_logits(logits))`` from a single pass over the logits, with
    a backward that writes the gradient of the logits once.  The reference calls the two functions back to back on the
    same logits (``verl/workers/engine/fsdp/transformer_impl.py:1400-1449``); as two autograd nodes each writes a full
    ``[rows, V]`` gradient and autograd adds them.  ``entropy_dtype``: dtype of the entropy (default: that of
    ``logits``; ``torch.float32`` gives what ``entropy_from_logits_with_chunking`` returns)."""
    return _LogprobsAndEntropyFromLogits.apply(logits, labels, logits.dtype if entropy_dtype is None else entropy_dtype)


def logprobs_from_logits(logits, labels, inplace_backward=True):
    """log_softmax(logits)[label]; shape ``logits.shape[:-1]``, dtype of ``logits``.
    ``inplace_backward`` is accepted for signature compatibility; the logits are never overwritten."""
    return _LogprobsFromLogits.apply(logits, labels)


def logprobs_from_logits_flash_attn(logits, labels, inplace_backward=True):
    """The reference routes here when flash-attn's cross-entropy is importable; same value, same kernel
    (the ``torch_npu`` twin of the reference, :136-152, has no counterpart on this hardware)."""
    return _LogprobsFromLogits.apply(logits, labels)


def logprobs_from_logits_naive(logits, labels):
    return _LogprobsFromLogits.apply(logits, labels)


def logprobs_from_logits_v2(logits, labels):
    return _LogprobsFromLogits.apply(logits, labels)


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """logsumexp(logits) - sum(softmax(logits) * logits); dtype of ``logits``."""
    return _EntropyFromLogits.apply(logits, logits.dtype)


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048) -> torch.Tensor:
    """Same value, always fp32 like the reference's chunked variant; the kernel needs no chunking."""
    return _EntropyFromLogits.apply(logits, torch.float32)


class _SumPiSquaredFromLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits):
        rows, V = _as_rows(logits)
        R = rows.shape[0]
        dev = logits.device
        out = torch.empty((R,), device=dev, dtype=torch.float32)
        keep = ctx.needs_input_grad[0]
        lse = torch.empty((R,), device=dev, dtype=torch.float32) if keep else None
        if R > 0:
            with torch.cuda.device(dev):
                rc = _abi.load().lce_logits_sum_pi_squared(
                    rows.data_ptr(), rows.stride(0), R, V, _abi.dtype_code(logits.dtype), out.data_ptr(), _abi.ptr(lse), _abi.current_stream(dev)
                )
                _abi.check(rc, "lce_logits_sum_pi_squared")
        if keep:
            ctx.save_for_backward(rows, lse, out)
            ctx.shape, ctx.dtype = logits.shape, logits.dtype
        return out.reshape(logits.shape[:-1]).to(logits.dtype)

    @staticmethod
    def backward(ctx, g):
        rows, lse, s = ctx.saved_tensors
        R, V = rows.shape
        d = torch.empty((R, V), device=rows.device, dtype=rows.dtype)
        g = g.reshape(-1).to(torch.float32).contiguous()
        if R > 0:
            with torch.cuda.device(rows.device):
                rc = _abi.load().lce_logits_sum_pi_squared_backward(
                    rows.data_ptr(), rows.stride(0), R, V, _abi.dtype_code(rows.dtype), lse.data_ptr(), s.data_ptr(), g.data_ptr(),
                    d.data_ptr(), d.stride(0), _abi.current_stream(rows.device),
                )  # fmt: skip
                _abi.check(rc, "lce_logits_sum_pi_squared_backward")
        return d.reshape(ctx.shape).to(ctx.dtype)


def calculate_sum_pi_squared_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """sum over the vocabulary of softmax(logits)**2 = exp(logsumexp(2*logits) - 2*logsumexp(logits));
    shape ``logits.shape[:-1]``, dtype of ``logits``.  One pass over the logits.  Differentiable like the reference's
    plain-torch expression (``verl/utils/torch_functional.py:687-703``; the reference itself only calls it without a
    graph): the backward is one more pass, ``d_logits = g * 2 p (p - sum p**2)``."""
    _require_gpu(logits)
    return _SumPiSquaredFromLogits.apply(logits)


def masked_sum(values, mask, axis=None):
    valid_values = torch.where(mask.bool(), values, 0.0)
    return (valid_values * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None):
    s = masked_sum(values, mask, axis)
    return s / (mask.sum(axis=axis) + 1e-8)
