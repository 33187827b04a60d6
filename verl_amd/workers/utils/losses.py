"""Fused PPO actor loss on the fused head's outputs.

One HIP pass computes what the reference assembles from ``compute_policy_loss_vanilla`` + ``agg_loss``, ``kl_penalty``
and the entropy and KL terms of ``ppo_loss`` (``verl/trainer/ppo/core_algos.py:1140-1206,1286-1376,2188-2251``,
``verl/workers/utils/losses.py:57-155``) for the vanilla loss under any of ``agg_loss``'s aggregation modes, together
with the gradients w.r.t. ``log_prob`` and ``entropy``, so the backward of ``linear_cross_entropy`` starts from two
ready vectors instead of an elementwise autograd graph.  Metric names are the reference's.
"""

from __future__ import annotations

from typing import Optional

import torch

from ... import _abi


AGG_MODES = {
    "token-mean": 0,
    "token-sum": 1,
    "seq-mean-token-sum": 2,
    "seq-mean-token-sum-norm": 3,
    "seq-mean-token-mean": 4,
}

# kl_penalty's estimators (core_algos.py:2228-2245); a trailing "+" selects the straight-through variant (:2201-2213)
KL_TYPES = {"kl": 1, "k1": 1, "abs": 2, "mse": 3, "k2": 3, "low_var_kl": 4, "k3": 4}
KL_STRAIGHT_THROUGH = 16


def kl_type_number(kl_penalty: str) -> int:
    base = kl_penalty[:-1] if kl_penalty.endswith("+") else kl_penalty
    if base not in KL_TYPES:
        raise NotImplementedError(f"kl_penalty {kl_penalty!r}")  # core_algos.py:2247-2251 ("full" included)
    return KL_TYPES[base] | (KL_STRAIGHT_THROUGH if kl_penalty.endswith("+") else 0)


def agg_numbers(loss_agg_mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor):
    """agg_loss's arguments as the C ABI takes them; raises what the reference raises (core_algos.py:1172-1204)."""
    if loss_agg_mode not in AGG_MODES:
        raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")
    if dp_size > 1:
        if loss_agg_mode == "token-mean" and batch_num_tokens is None:
            raise ValueError("(global) batch_num_tokens is required when dp_size > 1")
        if loss_agg_mode.startswith("seq-mean") and global_batch_size is None:
            raise ValueError("global_batch_size is required when dp_size > 1")
    return (
        AGG_MODES[loss_agg_mode],
        float(dp_size),
        -1.0 if batch_num_tokens is None else float(batch_num_tokens),
        -1.0 if global_batch_size is None else float(global_batch_size),
        -1.0 if loss_scale_factor is None else float(loss_scale_factor),
    )


class _FusedPPOLoss(torch.autograd.Function):
    """``log_prob`` may be None: then the call is ``agg_loss`` of ``entropy`` (the C ABI's aggregation-only form)."""

    @staticmethod
    def forward(ctx, log_prob, entropy, old_log_prob, advantages, response_mask, is_weights, ref_log_prob, agg, kl,
                clip_low, clip_high, clip_c, entropy_coeff, packed=None):
        if packed is not None:
            return _FusedPPOLoss._forward_packed(ctx, log_prob, entropy, old_log_prob, advantages, response_mask, is_weights,
                                                 ref_log_prob, agg, kl, clip_low, clip_high, clip_c, entropy_coeff, packed)
        lead = log_prob if log_prob is not None else entropy
        assert lead.is_cuda, "fused_ppo_loss runs on the GPU only"
        dev = lead.device
        shape = lead.shape

        def f32(t):
            return None if t is None else t.detach().reshape(-1).to(torch.float32).contiguous()

        lp, ent, old, adv, mask = f32(log_prob), f32(entropy), f32(old_log_prob), f32(advantages), f32(response_mask)
        isw, ref = f32(is_weights), f32(ref_log_prob)
        n = lead.numel()
        for t in (lp, ent, old, adv, mask, isw, ref):
            assert t is None or t.numel() == n, "all inputs have the shape of log_prob"
        # rows are the sequences the seq-mean modes average over: the last dimension is the response
        row_len = shape[-1] if len(shape) >= 1 else 1
        rows = n // row_len if row_len else 0
        mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor = agg
        kl_type, kl_coef = kl
        out = torch.empty(16, device=dev, dtype=torch.float32)
        g_lp = None if lp is None else torch.empty(n, device=dev, dtype=torch.float32)
        g_ent = None if ent is None else torch.empty(n, device=dev, dtype=torch.float32)
        lib = _abi.load()
        with torch.cuda.device(dev):
            ws_bytes = lib.lce_ppo_loss_workspace_bytes(rows, row_len)
            ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
            rc = lib.lce_ppo_loss(
                _abi.ptr(lp), _abi.ptr(ent), _abi.ptr(old), _abi.ptr(adv), mask.data_ptr(), _abi.ptr(isw),
                _abi.ptr(ref), kl_type, kl_coef, rows, row_len, mode, clip_low, clip_high, clip_c, entropy_coeff,
                dp_size, batch_num_tokens, global_batch_size, loss_scale_factor, out.data_ptr(), _abi.ptr(g_lp),
                _abi.ptr(g_ent), ws.data_ptr(), ws_bytes, _abi.current_stream(dev),
            )  # fmt: skip
            _abi.check(rc, "lce_ppo_loss")
        empty = out.new_empty(0)
        ctx.save_for_backward(g_lp if g_lp is not None else empty, g_ent if g_ent is not None else empty)
        ctx.has = (lp is not None, ent is not None)
        ctx.shape = shape
        ctx.dtypes = (None if log_prob is None else log_prob.dtype, None if entropy is None else entropy.dtype)
        ctx.mark_non_differentiable(out)
        return out[0], out

    @staticmethod
    def _forward_packed(ctx, log_prob, entropy, old_log_prob, advantages, response_mask, is_weights, ref_log_prob, agg, kl,
                        clip_low, clip_high, clip_c, entropy_coeff, packed):
        """log_prob / entropy are [total_nnz] model outputs over the packed sequences; everything else is
        [batch, max_response_len]; packed = (response_start, response_len) int64 [batch] on the device."""
        assert log_prob is not None and log_prob.is_cuda, "fused_ppo_loss_packed runs on the GPU only"
        dev = log_prob.device
        start, length = packed
        rows, row_len = response_mask.shape
        total = log_prob.numel()

        def f32(t, n):
            if t is None:
                return None
            t = t.detach().reshape(-1).to(torch.float32).contiguous()
            assert t.numel() == n
            return t

        lp, ent = f32(log_prob, total), f32(entropy, total)
        old, adv, mask = f32(old_log_prob, rows * row_len), f32(advantages, rows * row_len), f32(response_mask, rows * row_len)
        isw, ref = f32(is_weights, rows * row_len), f32(ref_log_prob, rows * row_len)
        mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor = agg
        kl_type, kl_coef = kl
        out = torch.empty(16, device=dev, dtype=torch.float32)
        g_lp = torch.empty(total, device=dev, dtype=torch.float32)
        g_ent = None if ent is None else torch.empty(total, device=dev, dtype=torch.float32)
        lib = _abi.load()
        with torch.cuda.device(dev):
            ws_bytes = lib.lce_ppo_loss_workspace_bytes(rows, row_len)
            ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
            rc = lib.lce_ppo_loss_packed(
                lp.data_ptr(), _abi.ptr(ent), total, start.data_ptr(), length.data_ptr(), old.data_ptr(), adv.data_ptr(),
                mask.data_ptr(), _abi.ptr(isw), _abi.ptr(ref), kl_type, kl_coef, rows, row_len, mode, clip_low, clip_high, clip_c,
                entropy_coeff, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor, out.data_ptr(), g_lp.data_ptr(),
                _abi.ptr(g_ent), ws.data_ptr(), ws_bytes, _abi.current_stream(dev),
            )  # fmt: skip
            _abi.check(rc, "lce_ppo_loss_packed")
        empty = out.new_empty(0)
        ctx.save_for_backward(g_lp, g_ent if g_ent is not None else empty)
        ctx.has = (True, ent is not None)
        ctx.shape = log_prob.shape
        ctx.dtypes = (log_prob.dtype, None if entropy is None else entropy.dtype)
        ctx.mark_non_differentiable(out)
        return out[0], out

    @staticmethod
    def backward(ctx, g_loss, _g_out):
        g_lp, g_ent = ctx.saved_tensors
        d_lp = (g_lp * g_loss).reshape(ctx.shape).to(ctx.dtypes[0]) if ctx.has[0] else None
        d_ent = (g_ent * g_loss).reshape(ctx.shape).to(ctx.dtypes[1]) if ctx.has[1] else None
        return (d_lp, d_ent) + (None,) * 12


def fused_ppo_loss(
    log_prob: torch.Tensor,
    entropy: Optional[torch.Tensor],
    old_log_prob: torch.Tensor,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    clip_ratio: float = 0.2,
    clip_ratio_low: Optional[float] = None,
    clip_ratio_high: Optional[float] = None,
    clip_ratio_c: float = 3.0,
    entropy_coeff: float = 0.0,
    loss_agg_mode: str = "token-mean",
    dp_size: int = 1,
    batch_num_tokens: Optional[int] = None,
    global_batch_size: Optional[int] = None,
    loss_scale_factor: Optional[int] = None,
    rollout_is_weights: Optional[torch.Tensor] = None,
    ref_log_prob: Optional[torch.Tensor] = None,
    kl_loss_coef: float = 0.001,
    kl_loss_type: str = "low_var_kl",
    _packed=None,
):
    """Returns ``(policy_loss, metrics)``: ``policy_loss = pg_loss - entropy_coeff * entropy_loss
    [+ kl_loss_coef * kl_loss]`` (a 0-dim tensor with autograd), ``metrics`` a dict of 0-dim tensors under the
    reference's keys (no host sync is forced).
    ``dp_size``, ``batch_num_tokens``, ``global_batch_size`` and ``loss_scale_factor`` are ``agg_loss``'s
    (``core_algos.py:1140-1206``); the sequences of the ``seq-mean-*`` modes are the rows of the last dimension.
    ``rollout_is_weights`` multiplies the per-token policy loss (``core_algos.py:1362-1363``) and takes no gradient.
    With ``ref_log_prob`` the KL penalty of ``ppo_loss`` (``use_kl_loss``, ``losses.py:142-153``) is added:
    ``kl_loss_type`` is ``kl_penalty``'s estimator name, ``kl_loss_coef`` its weight."""
    agg = agg_numbers(loss_agg_mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor)
    assert clip_ratio_c > 1.0, f"clip_ratio_c must be greater than 1.0, got {clip_ratio_c}"
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    kl = (0, 0.0) if ref_log_prob is None else (kl_type_number(kl_loss_type), float(kl_loss_coef))
    loss, out = _FusedPPOLoss.apply(
        log_prob, entropy, old_log_prob, advantages, response_mask, rollout_is_weights, ref_log_prob, agg, kl,
        float(lo), float(hi), float(clip_ratio_c), float(entropy_coeff), _packed,
    )  # fmt: skip
    metrics = {
        "actor/pg_loss": out[1],
        "actor/pg_clipfrac": out[3],
        "actor/ppo_kl": out[4],
        "actor/pg_clipfrac_lower": out[5],
    }
    if entropy is not None:
        metrics["actor/entropy_loss"] = out[2]
    if ref_log_prob is not None:
        metrics["kl_loss"] = out[8]
        metrics["kl_coef"] = kl_loss_coef
    return loss, metrics


def response_slices(prompt_lens: torch.Tensor, response_lens: torch.Tensor, total_nnz: int):
    """``(start, length)`` per sequence of the response slice that ``no_padding_2_padding`` takes out of a packed model
    output (``verl/workers/utils/padding.py:97-141``): ``start = end of the sequence - response length - 1`` (the
    left shift by one token), with the reference's two assertions."""
    prompt_lens = prompt_lens.to(torch.int64)
    response_lens = response_lens.to(torch.int64)
    sequence_offsets = (prompt_lens + response_lens).cumsum(dim=0)
    assert sequence_offsets[-1].item() == total_nnz
    assert not prompt_lens.eq(0).any(), f"seq_offset - resp_len - 1 assumes prompt_len > 0. Got {prompt_lens}"
    return (sequence_offsets - response_lens - 1).contiguous(), response_lens.contiguous()


def fused_ppo_loss_packed(
    log_prob: torch.Tensor,
    entropy: Optional[torch.Tensor],
    prompt_lens: torch.Tensor,
    response_lens: torch.Tensor,
    old_log_prob: torch.Tensor,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    **kwargs,
):
    """``fused_ppo_loss`` for the no-padding engines: ``log_prob`` / ``entropy`` are the fused head's outputs over the
    PACKED sequences, ``[total_nnz]``; ``prompt_lens`` / ``response_lens`` ``[batch]`` (integer tensors on the device);
    ``old_log_prob``, ``advantages``, ``response_mask`` (and ``rollout_is_weights``, ``ref_log_prob``) stay
    ``[batch, max_response_len]`` as the data batch holds them.  The kernel applies the response slice of
    ``no_padding_2_padding`` (``verl/workers/utils/padding.py:97-141``) while it reads, and the gradients flow back in
    packed order, so the backward of ``linear_cross_entropy`` starts from them without a gather or a scatter.
    Same keyword arguments, return values and metrics as ``fused_ppo_loss``."""
    assert log_prob.dim() == 1 and (entropy is None or entropy.shape == log_prob.shape), "packed outputs are [total_nnz]"
    assert response_mask.dim() == 2 and old_log_prob.shape == response_mask.shape == advantages.shape
    assert prompt_lens.shape == response_lens.shape == (response_mask.shape[0],)
    dev = log_prob.device
    start, length = response_slices(prompt_lens.to(dev), response_lens.to(dev), log_prob.numel())
    assert int(length.max().item()) <= response_mask.shape[1], "a response is longer than max_response_len"
    return fused_ppo_loss(log_prob, entropy, old_log_prob, advantages, response_mask, _packed=(start, length), **kwargs)


def _cfg(config, name, default=None):
    """``config.name`` or ``config[name]``: the reference's configs are dataclasses that also answer ``.get``."""
    if isinstance(config, dict):
        return config.get(name, default)
    if hasattr(config, name):
        return getattr(config, name)
    return config.get(name, default) if hasattr(config, "get") else default


def _get(data, key, default=None):
    try:
        return data[key]
    except KeyError:
        return default


def _has(data, key) -> bool:
    try:
        return key in data
    except TypeError:
        return _get(data, key) is not None


def batch_lens(data):
    """``(prompt_lens, response_lens)`` of a data batch the way ``no_padding_2_padding`` reads them
    (``verl/workers/utils/padding.py:110-124``): from the offsets of nested ``prompts`` / ``responses``, or from the
    two halves of ``attention_mask`` when the batch is padded."""
    prompts, responses = data["prompts"], data["responses"]
    if prompts.is_nested:
        return prompts.offsets().diff(), responses.offsets().diff()
    attention_mask = data["attention_mask"]
    assert not attention_mask.is_nested
    P = prompts.shape[1]
    return attention_mask[:, :P].sum(dim=1), attention_mask[:, P:].sum(dim=1)


def _padded(t: torch.Tensor, width: int) -> torch.Tensor:
    """A batch field as exactly ``[batch, width]``: nested (jagged) fields are padded with zeros like
    ``to_padded_tensor``, then cut or zero-padded to ``width`` (a jagged tensor without a cached longest row can come
    back wider than its longest row; columns beyond every row's length hold padding only)."""
    if t.is_nested:
        t = torch.nested.to_padded_tensor(t, 0.0)
    if t.shape[1] > width:
        t = t[:, :width]
    elif t.shape[1] < width:
        t = torch.nn.functional.pad(t, (0, width - t.shape[1]))
    return t.contiguous()


def response_width(data, response_lens) -> int:
    """Padded width of the response slice as ``no_padding_2_padding`` picks it (``verl/workers/utils/padding.py:112-124``):
    for nested batches the non-tensor entry ``max_response_len`` when it is there and not negative, else the longest
    response; for padded batches the width of ``responses``."""
    responses = data["responses"]
    if not responses.is_nested:
        return int(responses.shape[1])
    given = _get(data, "max_response_len")
    given = getattr(given, "data", given)  # (a tensordict NonTensorData wraps its payload)
    if given is not None and int(given) >= 0:
        return int(given)
    return int(response_lens.max().item())


def metric_aggregation_for(dp_size, batch_num_tokens, global_batch_size, loss_scale_factor):
    """``losses.py:71-84``: once any global normaliser is set the loss of a micro-batch is already a share of the
    global mean, so its metric adds up over micro-batches (SUM); otherwise each is a local mean (MEAN)."""
    from ...utils.metric import AggregationType

    if dp_size > 1 or batch_num_tokens is not None or global_batch_size is not None or loss_scale_factor is not None:
        return AggregationType.SUM
    return AggregationType.MEAN


def ppo_loss(config, model_output, data, dp_group=None):
    """The reference's actor loss entry (``verl/workers/utils/losses.py:57-155``) on the fused kernels: same arguments,
    same ``(policy_loss, metrics)`` with ``Metric`` values under the reference's keys and aggregation kinds.

    ``model_output["log_probs"]`` / ``["entropy"]``: the head's outputs over the packed sequences (``[total_nnz]`` or
    nested); ``data``: a mapping with ``prompts``, ``responses`` (nested, or padded together with
    ``attention_mask``), ``response_mask``, ``old_log_probs``, ``advantages``, optionally ``rollout_is_weights`` and
    ``ref_log_prob``, and the entries ``dp_size``, ``batch_num_tokens``, ``global_batch_size``.  ``config``: an
    ``ActorConfig``-like object (``clip_ratio*``, ``entropy_coeff``, ``loss_agg_mode``, ``loss_scale_factor``,
    ``use_kl_loss``, ``kl_loss_coef``, ``kl_loss_type``, ``policy_loss.loss_mode``, dict ``global_batch_info``).
    The response slice, the policy loss, the entropy and KL terms and all metrics are ONE ``lce_ppo_loss_packed``
    call; gradients come back in packed order.  Only ``loss_mode == "vanilla"`` has a fused kernel; other modes and
    the sampler-correction outputs (``sc_*``) raise ``NotImplementedError`` instead of taking a slower path."""
    from ...utils.metric import AggregationType, Metric

    for key in ("sc_correction", "sc_sampler_head_mass", "sc_train_head_mass"):
        if _has(model_output, key):
            raise NotImplementedError(f"model output {key!r}: the fused PPO loss has no sampler-correction term")
    loss_mode = _cfg(_cfg(config, "policy_loss", {}) or {}, "loss_mode", "vanilla")
    if loss_mode != "vanilla":
        raise NotImplementedError(f"policy loss mode {loss_mode!r}: only 'vanilla' has a fused kernel")

    log_prob = model_output["log_probs"]
    log_prob = log_prob.values() if log_prob.is_nested else log_prob
    entropy = _get(model_output, "entropy")
    if entropy is not None and entropy.is_nested:
        entropy = entropy.values()

    info = {
        "dp_size": data["dp_size"],
        "batch_num_tokens": data["batch_num_tokens"],
        "global_batch_size": data["global_batch_size"],
        "loss_scale_factor": _cfg(config, "loss_scale_factor"),
    }
    shared = _cfg(config, "global_batch_info")
    if isinstance(shared, dict):  # the reference leaves them on the config for the policy-loss function
        shared.update(info)
    metric_aggregation = metric_aggregation_for(**info)

    prompt_lens, response_lens = batch_lens(data)
    width = response_width(data, response_lens)
    if int(response_lens.max().item()) > width:
        raise ValueError(f"max_response_len = {width} is shorter than the longest response ({int(response_lens.max().item())})")
    response_mask = _padded(data["response_mask"], width).to(bool)
    use_kl = bool(_cfg(config, "use_kl_loss", False))
    is_weights = _get(data, "rollout_is_weights")
    policy_loss, m = fused_ppo_loss_packed(
        log_prob, entropy, prompt_lens, response_lens,
        _padded(data["old_log_probs"], width), _padded(data["advantages"], width), response_mask,
        clip_ratio=_cfg(config, "clip_ratio"),
        clip_ratio_low=_cfg(config, "clip_ratio_low"),
        clip_ratio_high=_cfg(config, "clip_ratio_high"),
        clip_ratio_c=_cfg(config, "clip_ratio_c", 3.0),
        entropy_coeff=_cfg(config, "entropy_coeff", 0.0) if entropy is not None else 0.0,
        loss_agg_mode=_cfg(config, "loss_agg_mode", "token-mean"),
        rollout_is_weights=None if is_weights is None else _padded(is_weights, width),
        ref_log_prob=_padded(data["ref_log_prob"], width) if use_kl else None,
        kl_loss_coef=_cfg(config, "kl_loss_coef", 0.001),
        kl_loss_type=_cfg(config, "kl_loss_type", "low_var_kl"),
        **info,
    )  # fmt: skip
    metrics = Metric.from_dict(
        {k: m[k] for k in ("actor/pg_clipfrac", "actor/ppo_kl", "actor/pg_clipfrac_lower")}, AggregationType.MEAN
    )
    metrics["actor/pg_loss"] = Metric(metric_aggregation, m["actor/pg_loss"])
    if entropy is not None:
        metrics["actor/entropy_loss"] = Metric(metric_aggregation, m["actor/entropy_loss"])
    if use_kl:
        metrics["kl_loss"] = Metric(metric_aggregation, m["kl_loss"])
        metrics["kl_coef"] = _cfg(config, "kl_loss_coef", 0.001)
    return policy_loss, metrics
