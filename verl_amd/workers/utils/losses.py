"""Fused PPO actor loss on the fused head's outputs.

One HIP pass computes what the reference assembles from ``compute_policy_loss_vanilla`` + ``agg_loss`` and
the entropy bonus in ``ppo_loss`` (``verl/trainer/ppo/core_algos.py:1140-1206,1286-1376``,
``verl/workers/utils/losses.py:57-140``) for the vanilla loss under any of ``agg_loss``'s aggregation modes, together
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


class _FusedPPOLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_prob, entropy, old_log_prob, advantages, response_mask, is_weights, agg, clip_low, clip_high,
                clip_c, entropy_coeff):
        assert log_prob.is_cuda, "fused_ppo_loss runs on the GPU only"
        dev = log_prob.device
        shape = log_prob.shape

        def f32(t):
            return t.detach().reshape(-1).to(torch.float32).contiguous()

        lp, old, adv, mask = f32(log_prob), f32(old_log_prob), f32(advantages), f32(response_mask)
        ent = None if entropy is None else f32(entropy)
        isw = None if is_weights is None else f32(is_weights)
        n = lp.numel()
        assert old.numel() == n and adv.numel() == n and mask.numel() == n and (ent is None or ent.numel() == n)
        assert isw is None or isw.numel() == n
        # rows are the sequences the seq-mean modes average over: the last dimension is the response
        row_len = shape[-1] if len(shape) >= 1 else 1
        rows = n // row_len if row_len else 0
        mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor = agg
        out = torch.empty(8, device=dev, dtype=torch.float32)
        g_lp = torch.empty(n, device=dev, dtype=torch.float32)
        g_ent = None if ent is None else torch.empty(n, device=dev, dtype=torch.float32)
        lib = _abi.load()
        with torch.cuda.device(dev):
            ws_bytes = lib.lce_ppo_loss_workspace_bytes(rows, row_len)
            ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
            rc = lib.lce_ppo_loss(
                lp.data_ptr(), _abi.ptr(ent), old.data_ptr(), adv.data_ptr(), mask.data_ptr(), _abi.ptr(isw), rows,
                row_len, mode, clip_low, clip_high, clip_c, entropy_coeff, dp_size, batch_num_tokens,
                global_batch_size, loss_scale_factor, out.data_ptr(), g_lp.data_ptr(), _abi.ptr(g_ent), ws.data_ptr(),
                ws_bytes, _abi.current_stream(dev),
            )  # fmt: skip
            _abi.check(rc, "lce_ppo_loss")
        ctx.save_for_backward(g_lp, g_ent if g_ent is not None else g_lp.new_empty(0))
        ctx.has_entropy = ent is not None
        ctx.shape = shape
        ctx.dtypes = (log_prob.dtype, None if entropy is None else entropy.dtype)
        ctx.mark_non_differentiable(out)
        return out[0], out

    @staticmethod
    def backward(ctx, g_loss, _g_out):
        g_lp, g_ent = ctx.saved_tensors
        d_lp = (g_lp * g_loss).reshape(ctx.shape).to(ctx.dtypes[0])
        d_ent = (g_ent * g_loss).reshape(ctx.shape).to(ctx.dtypes[1]) if ctx.has_entropy else None
        return d_lp, d_ent, None, None, None, None, None, None, None, None, None


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
):
    """Returns ``(policy_loss, metrics)``: ``policy_loss = pg_loss - entropy_coeff * entropy_loss`` (a 0-dim tensor
    with autograd), ``metrics`` a dict of 0-dim tensors under the reference's keys (no host sync is forced).
    ``dp_size``, ``batch_num_tokens``, ``global_batch_size`` and ``loss_scale_factor`` are ``agg_loss``'s
    (``core_algos.py:1140-1206``); the sequences of the ``seq-mean-*`` modes are the rows of the last dimension.
    ``rollout_is_weights`` multiplies the per-token policy loss (``core_algos.py:1362-1363``) and takes no gradient."""
    if loss_agg_mode not in AGG_MODES:
        raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")
    assert clip_ratio_c > 1.0, f"clip_ratio_c must be greater than 1.0, got {clip_ratio_c}"
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    if dp_size > 1:
        if loss_agg_mode == "token-mean" and batch_num_tokens is None:
            raise ValueError("(global) batch_num_tokens is required when dp_size > 1")
        if loss_agg_mode.startswith("seq-mean") and global_batch_size is None:
            raise ValueError("global_batch_size is required when dp_size > 1")
    agg = (
        AGG_MODES[loss_agg_mode],
        float(dp_size),
        -1.0 if batch_num_tokens is None else float(batch_num_tokens),
        -1.0 if global_batch_size is None else float(global_batch_size),
        -1.0 if loss_scale_factor is None else float(loss_scale_factor),
    )
    loss, out = _FusedPPOLoss.apply(
        log_prob, entropy, old_log_prob, advantages, response_mask, rollout_is_weights, agg, float(lo), float(hi),
        float(clip_ratio_c), float(entropy_coeff),
    )  # fmt: skip
    metrics = {
        "actor/pg_loss": out[1],
        "actor/pg_clipfrac": out[3],
        "actor/ppo_kl": out[4],
        "actor/pg_clipfrac_lower": out[5],
    }
    if entropy is not None:
        metrics["actor/entropy_loss"] = out[2]
    return loss, metrics
