"""Host launchers of the fused lm-head log-prob + entropy kernels.

Same names, argument meaning, return tuples and error behaviour as the reference's
``verl/utils/kernel/kernels.py`` (enums :102-156, ``Config`` :160-172, ``set_backward_method`` :175-180,
``efficient_entropy_forward`` :569-759, ``efficient_entropy_backward`` :1518-1729); the device work is
done by hand-written gfx950 kernels behind the C ABI of ``liblce_gfx950.so``.

Differences that are deliberate (all inside the reference's own tolerances):
* the per-token max is the true max of the logits (the reference seeds its merge with 0);
* ``d_hidden`` / ``d_weight`` are accumulated in fp32 over vocabulary chunks and rounded once;
* ``BackwardEnum`` values are accepted by ``set_backward_method`` but select nothing: there is one
  backward schedule (recompute a vocab-chunk of d_logits, then two MFMA GEMMs);
* labels outside ``[0, V)`` give ``logprob = -logsumexp`` instead of reading uninitialised memory;
* ``dist_process_group`` with more than one rank (vocab-parallel) raises ``NotImplementedError``; a group of one
  rank (what Megatron passes at tensor-parallel size 1, ``verl/models/mcore/model_forward_fused.py:110-117``) is the
  single-GPU path.
"""

from __future__ import annotations

import typing
from dataclasses import dataclass

import torch

from ... import _abi


@dataclass
class EntropyReductionEnum:
    _None = 0
    _Sum = 1
    _Mean = 2


def get_entropy_reduction_enum_number(reduction: str) -> int:
    if reduction == "none":
        return EntropyReductionEnum._None
    if reduction == "sum":
        return EntropyReductionEnum._Sum
    if reduction == "mean":
        return EntropyReductionEnum._Mean
    raise ValueError(f"Invalid reduction: {reduction}")


def get_entropy_reduction_enum(ce_reduction: int) -> int:
    if ce_reduction in (0, 1, 2):
        return ce_reduction
    raise ValueError(f"Invalid ce_reduction: {ce_reduction}")


@dataclass
class BackwardEnum:
    _Total_Fuse_MN = 0
    _Total_Separate = 1
    _Split_Dlogits_N = 2
    _Split_Dlogits_M = 3


@dataclass
class Config:
    _backward: int = BackwardEnum._Split_Dlogits_N
    _use_triton: bool = False  # kept for attribute compatibility; there is no Triton here
    _vocab_chunk: int = 0  # columns of d_logits alive at once in the backward (0 = library default)


_config = Config()


def set_backward_method(backward_method: int):
    """Accepted for compatibility; every method maps to the one HIP backward schedule."""
    global _config
    _config._backward = backward_method


def set_vocab_chunk(columns: int):
    """Vocabulary columns of d_logits materialised per backward step (multiple of 256; 0 = default)."""
    global _config
    _config._vocab_chunk = int(columns)


def set_workspace_budget(num_bytes: int):
    """Byte budget of the backward's workspace (process-wide; 0 = the library's default rule: chunks of 8192 vocabulary
    columns, wider while one d_logits buffer stays within 256 MiB).  The library then picks the widest vocabulary chunk
    whose workspace fits the budget (never fewer than 2048 columns) and never exceeds its own upper bound of a quarter of
    one ``[T, V]`` tensor plus one fp32 ``[V, H]``.  An explicit ``set_vocab_chunk`` takes precedence."""
    _abi.check(_abi.load().lce_set_option(8, int(num_bytes)), "lce_set_option")


def set_keep_logits_tokens(tokens: int | None):
    """Token count up to which ``linear_cross_entropy`` keeps its fp32 logits for the backward (process-wide), next to
    the library's own bound of half the hidden size.  ``None`` (the default setting): only that bound.  0: every
    backward recomputes them from ``hidden`` and ``weight``, as the reference does at every size."""
    _abi.check(_abi.load().lce_set_option(11, (1 << 40) if tokens is None else int(tokens)), "lce_set_option")


def _require_single_rank(dist_process_group) -> None:
    """The vocabulary is not sharded here: only ``None`` or a process group of exactly one rank is accepted."""
    if dist_process_group is None:
        return
    try:
        size = getattr(dist_process_group, "size", None)
        if callable(size):
            world = int(size())
        else:
            import torch.distributed as dist

            world = dist.get_world_size(dist_process_group)
    except Exception:
        world = -1  # not a process group
    if world != 1:
        raise NotImplementedError("vocab-parallel (dist_process_group) is not built: one GPU, no collectives")


def _check_inputs(hidden, weight, labels):
    assert hidden.is_cuda and weight.is_cuda and labels.is_cuda
    assert weight.device == hidden.device and labels.device == hidden.device
    assert hidden.dim() == 2 and weight.dim() == 2 and labels.dim() == 1
    assert hidden.is_contiguous() and weight.is_contiguous() and labels.is_contiguous()
    assert hidden.shape[0] == labels.shape[0] and hidden.shape[1] == weight.shape[1]
    assert hidden.shape[1] % 128 == 0
    if hidden.dtype != weight.dtype:
        raise NotImplementedError(f"hidden ({hidden.dtype}) and weight ({weight.dtype}) must share a dtype")
    if labels.dtype != torch.int64:
        raise NotImplementedError(f"labels must be int64, got {labels.dtype}")
    return _abi.dtype_code(hidden.dtype)


def efficient_entropy_forward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    reduction: typing.Optional[int] = 2,
    temperature: typing.Optional[float] = 1.0,
    dist_process_group=None,
) -> list[torch.Tensor]:
    """Returns (logprobs, entropy, maximum, accumulate, entropy_b), all fp32."""
    return forward_keeping_logits(hidden, weight, labels, reduction, temperature, dist_process_group, keep_logits=False)[:5]


def forward_keeping_logits(hidden, weight, labels, reduction=2, temperature=1.0, dist_process_group=None, *, keep_logits=True):
    """``efficient_entropy_forward`` plus a sixth value: the kept logits for ``efficient_entropy_backward(...,
    logits_cache=)``, or ``None`` where the library keeps none (more tokens than half the hidden size, fp32
    inputs, ``keep_logits=False``).
    With few tokens fp32 ``[T, V]`` is a fraction of the weight itself, so the autograd node keeps it like any activation
    and the backward skips the pass over ``[V, H]`` and the ``T x V x H`` product that recompute it (not in the
    reference, which always recomputes)."""
    _require_single_rank(dist_process_group)
    code = _check_inputs(hidden, weight, labels)
    reduction = get_entropy_reduction_enum(reduction)
    assert temperature > 0, "temperature must be positive"
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    f32 = dict(device=dev, dtype=torch.float32)
    logprobs = torch.empty((T,) if reduction == 0 else (), **f32)
    entropy = torch.empty((T,), **f32)
    maximum = torch.empty((T,), **f32)
    acc_eb = torch.empty((2, T), **f32)
    accumulate, entropy_b = acc_eb[0], acc_eb[1]
    if T == 0:
        if reduction != 0:
            logprobs.zero_()
        return logprobs, entropy, maximum, accumulate, entropy_b, None
    lib = _abi.load()
    cache = None
    with torch.cuda.device(dev):
        ws_bytes = lib.lce_forward_workspace_bytes(T, H, V, code)
        ws = torch.empty((ws_bytes,), device=dev, dtype=torch.uint8)
        cache_bytes = lib.lce_logits_cache_bytes(T, H, V, code) if keep_logits else 0
        if cache_bytes:
            cache = torch.empty((cache_bytes,), device=dev, dtype=torch.uint8)
        rc = lib.lce_forward_keep_logits(
            hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), labels.data_ptr(), T, H, V, code,
            float(temperature), reduction, logprobs.data_ptr(), entropy.data_ptr(), maximum.data_ptr(),
            accumulate.data_ptr(), entropy_b.data_ptr(), ws.data_ptr(), ws_bytes, _abi.ptr(cache), cache_bytes,
            _abi.current_stream(dev),
        )  # fmt: skip
        _abi.check(rc, "lce_forward_keep_logits")
    return logprobs, entropy, maximum, accumulate, entropy_b, cache


def efficient_entropy_backward(
    dlogprobs: torch.Tensor,
    dentropy: typing.Optional[torch.Tensor],
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    maximum: torch.Tensor,
    acc: torch.Tensor,
    entropy_b: torch.Tensor,
    reduction: typing.Optional[int] = 2,
    should_return_fp32_grad: bool = False,
    temperature: typing.Optional[float] = 1.0,
    dist_process_group=None,
    *,
    need_d_hidden: bool = True,
    need_d_weight: bool = True,
    logits_cache: typing.Optional[torch.Tensor] = None,
) -> list[torch.Tensor]:
    """Returns (d_hidden, d_weight) in ``hidden.dtype`` (fp32 when ``should_return_fp32_grad``).

    ``need_d_hidden`` / ``need_d_weight`` (not in the reference, which always computes both): ``False`` leaves that
    gradient's GEMM out, a third of the backward's work, and returns ``None`` in its place, e.g. for a frozen lm-head
    under LoRA.  ``logits_cache``: the sixth value of ``forward_keeping_logits`` for the same inputs; the gradients are
    bit for bit the same with and without it."""
    if not (need_d_hidden or need_d_weight):
        return None, None
    _require_single_rank(dist_process_group)
    if _config._backward == BackwardEnum._Split_Dlogits_M:
        raise NotImplementedError("BackwardEnum._Split_Dlogits_M is not implemented yet")
    code = _check_inputs(hidden, weight, labels)
    reduction = get_entropy_reduction_enum(reduction)
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    if reduction == 0:
        assert dlogprobs.shape == (T,)
    else:
        assert dlogprobs.dim() == 0
    assert dlogprobs.is_cuda and dlogprobs.device == dev
    assert maximum.shape == labels.shape == acc.shape and entropy_b.shape == (T,)
    assert maximum.is_contiguous() and acc.is_contiguous() and entropy_b.is_contiguous()
    g_lp = dlogprobs.detach().to(torch.float32).contiguous()
    g_ent = None
    if dentropy is not None:
        assert dentropy.is_cuda and dentropy.device == dev and dentropy.shape == (T,)
        g_ent = dentropy.detach().to(torch.float32).contiguous()
    # should_return_fp32_grad: both gradients straight from the fp32 accumulators, without the rounding to the input dtype
    # (verl/utils/kernel/kernels.py:1562-1567)
    grad_dtype = torch.float32 if should_return_fp32_grad else hidden.dtype
    d_hidden = torch.empty((T, H), device=dev, dtype=grad_dtype) if need_d_hidden else None
    d_weight = torch.empty((V, H), device=dev, dtype=grad_dtype) if need_d_weight else None
    if T == 0:
        if d_weight is not None:
            d_weight.zero_()
    else:
        lib = _abi.load()
        with torch.cuda.device(dev):
            vchunk = _config._vocab_chunk
            ws_bytes = lib.lce_backward_workspace_bytes(T, H, V, code, vchunk)
            ws = torch.empty((ws_bytes,), device=dev, dtype=torch.uint8)
            if logits_cache is not None:
                assert logits_cache.is_cuda and logits_cache.device == dev and logits_cache.is_contiguous()
                rc = lib.lce_backward_from_logits(
                    hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), labels.data_ptr(), T, H, V,
                    code, float(temperature), reduction, maximum.data_ptr(), acc.data_ptr(), entropy_b.data_ptr(),
                    g_lp.data_ptr(), _abi.ptr(g_ent), _abi.ptr(d_hidden), _abi.ptr(d_weight), int(should_return_fp32_grad),
                    ws.data_ptr(), ws_bytes, vchunk, logits_cache.data_ptr(), logits_cache.numel() * logits_cache.element_size(),
                    _abi.current_stream(dev),
                )  # fmt: skip
                _abi.check(rc, "lce_backward_from_logits")
                return d_hidden, d_weight
            entry = lib.lce_backward_f32 if should_return_fp32_grad else lib.lce_backward
            rc = entry(
                hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), labels.data_ptr(), T, H, V,
                code, float(temperature), reduction, maximum.data_ptr(), acc.data_ptr(), entropy_b.data_ptr(),
                g_lp.data_ptr(), _abi.ptr(g_ent), _abi.ptr(d_hidden), _abi.ptr(d_weight), ws.data_ptr(), ws_bytes,
                vchunk, _abi.current_stream(dev),
            )  # fmt: skip
            _abi.check(rc, "lce_backward")
    return d_hidden, d_weight
