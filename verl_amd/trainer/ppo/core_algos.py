"""The two functions of the reference's ``verl/trainer/ppo/core_algos.py`` that sit directly behind the fused head:
``agg_loss`` (``:1140-1206``) and ``compute_policy_loss_vanilla`` (``:1286-1376``; its deprecated predecessor
``compute_policy_loss``, ``:1210-1282``, and the registry lookup ``get_policy_loss_fn``, ``:70-85``), with the reference's names,
argument order and return values, computed by the HIP PPO-loss kernels (``lce_ppo_loss``).  Both are
differentiable; nothing here runs on the CPU."""

from __future__ import annotations

import warnings
from typing import Any, Optional

import torch

from ...workers.utils.losses import _cfg, _FusedPPOLoss, agg_numbers, fused_ppo_loss


def agg_loss(
    loss_mat: torch.Tensor,
    loss_mask: torch.Tensor,
    loss_agg_mode: str,
    dp_size: int = 1,
    batch_num_tokens: Optional[int] = None,
    global_batch_size: Optional[int] = None,
    loss_scale_factor: Optional[int] = None,
) -> torch.Tensor:
    """``loss_mat``, ``loss_mask`` ``[bs, response_length]`` -> scalar, in any of the five modes of the reference."""
    agg = agg_numbers(loss_agg_mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor)
    # aggregation-only form of the kernel: loss = 0 - (-1) * agg(loss_mat)
    loss, _ = _FusedPPOLoss.apply(None, loss_mat, None, None, loss_mask, None, None, agg, (0, 0.0), 0.2, 0.2, 3.0, -1.0)
    return loss


def compute_policy_loss_vanilla(
    old_log_prob: torch.Tensor,
    log_prob: torch.Tensor,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    loss_agg_mode: str = "token-mean",
    config: Optional[Any] = None,
    rollout_is_weights: torch.Tensor | None = None,
) -> tuple[torch.Tensor, dict[str, Any]]:
    """``config`` carries ``clip_ratio``, ``clip_ratio_low``, ``clip_ratio_high``, ``clip_ratio_c`` (default 3.0) and
    the dict ``global_batch_info`` (``dp_size``, ``batch_num_tokens``, ``global_batch_size``, ``loss_scale_factor``),
    as attributes or keys.  Returns ``(pg_loss, pg_metrics)`` with the metrics as Python floats, like the reference
    (which therefore synchronises; ``fused_ppo_loss`` returns them as device scalars instead)."""
    assert config is not None
    clip_ratio = _cfg(config, "clip_ratio")
    info = dict(_cfg(config, "global_batch_info", {}) or {})
    pg_loss, metrics = fused_ppo_loss(
        log_prob, None, old_log_prob, advantages, response_mask,
        clip_ratio=clip_ratio,
        clip_ratio_low=_cfg(config, "clip_ratio_low"),
        clip_ratio_high=_cfg(config, "clip_ratio_high"),
        clip_ratio_c=_cfg(config, "clip_ratio_c", 3.0),
        loss_agg_mode=loss_agg_mode,
        rollout_is_weights=rollout_is_weights,
        **info,
    )  # fmt: skip
    pg_metrics = {
        k: metrics[k].detach().item() for k in ("actor/pg_clipfrac", "actor/ppo_kl", "actor/pg_clipfrac_lower")
    }
    return pg_loss, pg_metrics


def compute_policy_loss(
    old_log_prob,
    log_prob,
    advantages,
    response_mask,
    cliprange=None,
    cliprange_low=None,
    cliprange_high=None,
    clip_ratio_c=3.0,
    loss_agg_mode: str = "token-mean",
):
    """Deprecated spelling of the vanilla loss (the reference warns with ``FutureWarning`` and so does this): no
    config object, no IS weights, no global normalisers; returns the 4-tuple ``(pg_loss, pg_clipfrac, ppo_kl,
    pg_clipfrac_lower)`` with the three statistics as 0-dim tensors, like the reference's ``masked_mean`` results."""
    warnings.warn(
        "Warning: Function 'verl_amd.trainer.ppo.core_algos.compute_policy_loss' is deprecated. Please use "
        "'verl_amd.trainer.ppo.core_algos.compute_policy_loss_vanilla' instead.",
        category=FutureWarning,
        stacklevel=2,
    )
    pg_loss, m = fused_ppo_loss(
        log_prob, None, old_log_prob, advantages, response_mask,
        clip_ratio=cliprange, clip_ratio_low=cliprange_low, clip_ratio_high=cliprange_high, clip_ratio_c=clip_ratio_c,
        loss_agg_mode=loss_agg_mode,
    )  # fmt: skip
    return pg_loss, m["actor/pg_clipfrac"], m["actor/ppo_kl"], m["actor/pg_clipfrac_lower"]


POLICY_LOSS_REGISTRY = {"vanilla": compute_policy_loss_vanilla}


def get_policy_loss_fn(name):
    """Only the vanilla loss has a fused kernel; the message is the reference's."""
    if name not in POLICY_LOSS_REGISTRY:
        raise ValueError(f"Unsupported loss mode: {name}. Supported modes are: {list(POLICY_LOSS_REGISTRY.keys())}")
    return POLICY_LOSS_REGISTRY[name]
