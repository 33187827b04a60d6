"""Per-rank pieces of a vocabulary-parallel (tensor-parallel) lm-head on one GPU.

The reference shards ``weight`` over the ranks of ``dist_process_group`` and exchanges per-token
statistics with three all-reduces (``verl/utils/kernel/kernels.py:705-757``, TP epilogue ``:444-566``);
labels stay global and are matched with the rank's vocabulary offset (``:328``, ``:1503``).  This module
holds what ONE rank computes, as thin wrappers over the C ABI:

* ``shard_forward``   -> partials ``[T, 4]`` = (max, sum exp, sum logit*exp, label logit or 0)
* ``merge_shards``    -> the five outputs of the unsharded forward from stacked partials ``[R, T, 4]``
* ``shard_backward``  -> (this shard's contribution to ``d_hidden``, ``d_weight`` of the shard)

The exchange itself (one all-gather of the partials, one sum of ``d_hidden``) belongs to the caller;
nothing here communicates.  ``linear_cross_entropy(..., dist_process_group=...)`` therefore still raises.
"""

from __future__ import annotations

import typing

import torch

from ... import _abi
from .kernels import _check_inputs, _config, get_entropy_reduction_enum, get_entropy_reduction_enum_number


def _reduction(reduction: typing.Union[int, str]) -> int:
    return get_entropy_reduction_enum_number(reduction) if isinstance(reduction, str) else get_entropy_reduction_enum(reduction)


def shard_forward(hidden: torch.Tensor, weight_shard: torch.Tensor, labels: torch.Tensor, vocab_offset: int,
                  temperature: float = 1.0) -> torch.Tensor:
    """Partial statistics of ``hidden @ weight_shard.T / temperature`` for global ``labels``."""
    code = _check_inputs(hidden, weight_shard, labels)
    assert temperature > 0 and vocab_offset >= 0
    T, H = hidden.shape
    V = weight_shard.shape[0]
    dev = hidden.device
    partials = torch.empty((T, 4), device=dev, dtype=torch.float32)
    if T == 0:
        return partials
    lib = _abi.load()
    with torch.cuda.device(dev):
        nws = lib.lce_forward_workspace_bytes(T, H, V, code)
        ws = torch.empty((nws,), device=dev, dtype=torch.uint8)
        rc = lib.lce_forward_shard(
            hidden.data_ptr(), hidden.stride(0), weight_shard.data_ptr(), weight_shard.stride(0), labels.data_ptr(), T, H, V,
            int(vocab_offset), code, float(temperature), partials.data_ptr(), ws.data_ptr(), nws, _abi.current_stream(dev),
        )  # fmt: skip
        _abi.check(rc, "lce_forward_shard")
    return partials


def merge_shards(partials: torch.Tensor, reduction: typing.Union[int, str] = 0) -> list[torch.Tensor]:
    """``partials [R, T, 4]`` (shard-major, as an all-gather delivers them) ->
    (logprobs, entropy, maximum, accumulate, entropy_b) of the whole vocabulary, fp32."""
    assert partials.is_cuda and partials.dtype == torch.float32 and partials.dim() == 3 and partials.shape[2] == 4
    partials = partials.contiguous()
    reduction = _reduction(reduction)
    R, T, _ = partials.shape
    dev = partials.device
    f32 = dict(device=dev, dtype=torch.float32)
    logprobs = torch.empty((T,) if reduction == 0 else (), **f32)
    entropy, maximum, accumulate, entropy_b = (torch.empty((T,), **f32) for _ in range(4))
    lib = _abi.load()
    with torch.cuda.device(dev):
        ws = torch.empty((max(4 * T, 16),), device=dev, dtype=torch.uint8)
        rc = lib.lce_merge_shards(
            partials.data_ptr(), R, T, reduction, logprobs.data_ptr(), entropy.data_ptr(), maximum.data_ptr(),
            accumulate.data_ptr(), entropy_b.data_ptr(), ws.data_ptr(), ws.numel(), _abi.current_stream(dev),
        )  # fmt: skip
        _abi.check(rc, "lce_merge_shards")
    return [logprobs, entropy, maximum, accumulate, entropy_b]


def shard_backward(dlogprobs: torch.Tensor, dentropy: typing.Optional[torch.Tensor], hidden: torch.Tensor,
                   weight_shard: torch.Tensor, labels: torch.Tensor, vocab_offset: int, maximum: torch.Tensor,
                   accumulate: torch.Tensor, entropy_b: torch.Tensor, reduction: typing.Union[int, str] = 0,
                   temperature: float = 1.0) -> list[torch.Tensor]:
    """(d_hidden contribution of this shard ``[T, H]``, d_weight of the shard ``[V_local, H]``), both in
    ``hidden.dtype``; ``maximum / accumulate / entropy_b`` are the MERGED statistics."""
    code = _check_inputs(hidden, weight_shard, labels)
    reduction = _reduction(reduction)
    T, H = hidden.shape
    V = weight_shard.shape[0]
    dev = hidden.device
    g_lp = dlogprobs.detach().to(torch.float32).contiguous()
    assert g_lp.shape == ((T,) if reduction == 0 else ())
    g_ent = None if dentropy is None else dentropy.detach().to(torch.float32).contiguous()
    d_hidden = torch.empty_like(hidden)
    d_weight = torch.empty((V, H), device=dev, dtype=hidden.dtype)
    if T == 0:
        d_weight.zero_()
        return [d_hidden, d_weight]
    lib = _abi.load()
    with torch.cuda.device(dev):
        vchunk = _config._vocab_chunk
        nws = lib.lce_backward_workspace_bytes(T, H, V, code, vchunk)
        ws = torch.empty((nws,), device=dev, dtype=torch.uint8)
        rc = lib.lce_backward_shard(
            hidden.data_ptr(), hidden.stride(0), weight_shard.data_ptr(), weight_shard.stride(0), labels.data_ptr(), T, H, V,
            int(vocab_offset), code, float(temperature), reduction, maximum.data_ptr(), accumulate.data_ptr(),
            entropy_b.data_ptr(), g_lp.data_ptr(), _abi.ptr(g_ent), d_hidden.data_ptr(), d_weight.data_ptr(), ws.data_ptr(),
            nws, vchunk, _abi.current_stream(dev),
        )  # fmt: skip
        _abi.check(rc, "lce_backward_shard")
    return [d_hidden, d_weight]
