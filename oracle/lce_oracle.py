"""CPU restatement of the lm-head log-prob + entropy path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it exists so that tests, the smoke check
and the benchmark's CPU-baseline leg have an independent statement of what the HIP kernels must
compute.  It materialises logits (chunked over tokens so any size fits in host memory) and uses
only torch library routines, evaluated in fp32 or fp64 on whatever inputs it is given.

What each function follows in the reference tree (paths relative to the reference root):

* ``lce_forward``            tests/utils/test_linear_cross_entropy.py:49-62 (``run_torch_entropy``),
                             verl/utils/kernel/kernels.py:306-329,419-433 (scale after the GEMM,
                             ``entropy = log(accu) + max - b``, ``logprob = label_logit - lse``)
* ``lce_backward``           verl/utils/kernel/kernels.py:1443-1507 (closed-form ``d_logits``),
                             :1714-1724 (``d_hidden = dz @ W``, ``d_weight = dz.T @ h``),
                             verl/utils/experimental/torch_functional.py:61-93 (same math)
* ``lce_unfused_autograd``   tests/utils/test_linear_cross_entropy.py:49-62 with ``torch.autograd.grad`` (:254-262): the
                             same values once more through autograd on materialised logits (pinned by equality
                             with ``lce_forward`` / ``lce_backward``)
* ``logprobs_from_logits``   verl/utils/torch_functional.py:155-207
* ``entropy_from_logits``    verl/utils/torch_functional.py:231-245
* ``sum_pi_squared_from_logits`` verl/utils/torch_functional.py:687-703
* ``logits_backward``        autograd of the two functions above, spelled out
* ``masked_sum/masked_mean`` verl/utils/torch_functional.py:273-308
* ``agg_loss``               verl/trainer/ppo/core_algos.py:1140-1206
* ``policy_loss_vanilla``    verl/trainer/ppo/core_algos.py:1286-1376
* ``kl_penalty``             verl/trainer/ppo/core_algos.py:2188-2251
* ``ppo_actor_loss``         verl/workers/utils/losses.py:57-153 (policy loss minus entropy bonus plus KL penalty)
* ``no_padding_2_padding``   verl/workers/utils/padding.py:97-141 (response slice of a packed model output)

How each is pinned (see tests/test_oracle_*.py): the reference's own known-answer vector for the
padded-vocab regression (tests/utils/test_linear_cross_entropy.py:352-395, closed form
``3 - log(e^3 + (V-1)e^-15)``), uniform-logit closed forms (entropy ``log V``), shift invariance,
fp64 brute force in pure Python on tiny inputs, ``torch.autograd`` and central finite differences
for the gradients, the invariant ``sum_v dz = 0``, for ``sum_pi_squared_from_logits`` the closed forms
``1/V`` (uniform), ``(1 + (V-1) r^2) / (1 + (V-1) r)^2`` (one logit raised by ``log(1/r)``) and a pure-Python
``sum(softmax**2)``, the independent C restatement in
``lce_oracle.c``, and the reference's known answers for ``agg_loss`` / ``masked_mean``
(tests/trainer/ppo/test_loss_aggregation_on_cpu.py:23-65, tests/utils/test_torch_functional.py:61-72);
``kl_penalty`` by its definitions evaluated with ``math.exp`` on scalars, ``k3 >= 0``, ``k3 = d^2/2 + O(d^3)``,
``E_pi[k1] = E_pi[k3] = KL`` on a small categorical distribution and autograd for the straight-through variants;
``no_padding_2_padding`` by a packed batch written out by hand (response lengths 3, 1 and 0) and the reference's two assertions.
No function here is "parity unpinned".
"""

from __future__ import annotations

import math
from typing import Optional

import torch

_REDUCTIONS = ("none", "sum", "mean")


def _check_reduction(reduction: str) -> str:
    reduction = reduction.lower()
    if reduction not in _REDUCTIONS:
        raise ValueError(f"Invalid reduction: {reduction}")
    return reduction


def _flatten(hidden: torch.Tensor, labels: torch.Tensor):
    return hidden.reshape(-1, hidden.shape[-1]), labels.reshape(-1).long()


def lce_forward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    reduction: str = "none",
    compute_dtype: torch.dtype = torch.float32,
    chunk: int = 1024,
    return_stats: bool = False,
):
    """logits = (h @ W^T) / tau in ``compute_dtype``; logprob = log_softmax(logits)[label];
    entropy = logsumexp(logits) - sum(softmax(logits) * logits).  Outputs are flattened [T]."""
    reduction = _check_reduction(reduction)
    h2, y = _flatten(hidden, labels)
    T = h2.shape[0]
    w = weight.to(compute_dtype)
    logprobs = torch.empty(T, dtype=compute_dtype, device=h2.device)
    entropy = torch.empty_like(logprobs)
    mx = torch.empty_like(logprobs)
    acc = torch.empty_like(logprobs)
    eb = torch.empty_like(logprobs)
    for s in range(0, T, chunk):
        e = min(T, s + chunk)
        z = h2[s:e].to(compute_dtype) @ w.t()
        z /= temperature
        lse = torch.logsumexp(z, dim=-1)
        pd = torch.softmax(z, dim=-1)
        b = torch.sum(pd * z, dim=-1)
        entropy[s:e] = lse - b
        logprobs[s:e] = torch.gather(z, -1, y[s:e].unsqueeze(-1)).squeeze(-1) - lse
        m = z.max(dim=-1).values
        mx[s:e] = m
        acc[s:e] = torch.exp(z - m.unsqueeze(-1)).sum(-1)
        eb[s:e] = b
    if reduction == "sum":
        logprobs = logprobs.sum()
    elif reduction == "mean":
        logprobs = logprobs.sum() / T
    if return_stats:
        return logprobs, entropy, mx, acc, eb
    return logprobs, entropy


def lce_backward(
    dlogprobs: torch.Tensor,
    dentropy: Optional[torch.Tensor],
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    reduction: str = "none",
    compute_dtype: torch.dtype = torch.float32,
    chunk: int = 1024,
):
    """dz = g_lp * (onehot - p) - g_ent * p * (z - b), then dz /= tau;
    d_hidden = dz @ W, d_weight = dz^T @ h.  Returned in ``compute_dtype``."""
    reduction = _check_reduction(reduction)
    h2, y = _flatten(hidden, labels)
    T = h2.shape[0]
    w = weight.to(compute_dtype)
    if reduction == "none":
        g_lp = dlogprobs.reshape(-1).to(compute_dtype)
    elif reduction == "sum":
        g_lp = dlogprobs.to(compute_dtype).reshape(()).expand(T)
    else:
        g_lp = (dlogprobs.to(compute_dtype).reshape(()) / T).expand(T)
    g_ent = None if dentropy is None else dentropy.reshape(-1).to(compute_dtype)
    d_hidden = torch.empty(h2.shape, dtype=compute_dtype, device=h2.device)
    d_weight = torch.zeros(w.shape, dtype=compute_dtype, device=w.device)
    for s in range(0, T, chunk):
        e = min(T, s + chunk)
        hc = h2[s:e].to(compute_dtype)
        z = hc @ w.t()
        z /= temperature
        p = torch.softmax(z, dim=-1)
        b = torch.sum(p * z, dim=-1, keepdim=True)
        dz = -p * g_lp[s:e].unsqueeze(-1)
        dz.scatter_add_(-1, y[s:e].unsqueeze(-1), g_lp[s:e].unsqueeze(-1).clone())
        if g_ent is not None:
            dz -= g_ent[s:e].unsqueeze(-1) * p * (z - b)
        dz /= temperature
        d_hidden[s:e] = dz @ w
        d_weight += dz.t() @ hc
    return d_hidden.reshape(hidden.shape), d_weight


def lce_unfused_autograd(hidden, weight, labels, temperature, g_logprobs, g_entropy, compute_dtype=torch.float32):
    """The unfused path exactly as the reference's test states it (tests/utils/test_linear_cross_entropy.py:49-62,
    ``run_torch_entropy``): one materialised ``[T, V]`` logits tensor in ``compute_dtype``, ``softmax``,
    ``logsumexp``, ``cross_entropy``, gradients by ``torch.autograd.grad``.  Returns
    ``(logprobs, entropy, d_hidden, d_weight)``; checked against ``lce_forward`` / ``lce_backward`` (the chunked closed
    form) in tests/test_oracle_lce.py.  The benchmark times it on the GPU as the context figure the reference's test
    prints next to its fused kernel (:290-349); it is never the product path."""
    h = hidden.detach().reshape(-1, hidden.shape[-1]).requires_grad_(True)
    w = weight.detach().requires_grad_(True)
    logits = torch.matmul(h.to(compute_dtype), w.to(compute_dtype).transpose(0, 1))
    logits = logits / temperature
    pd = torch.nn.functional.softmax(logits, dim=-1)
    entropy = torch.logsumexp(logits, dim=-1) - torch.sum(pd * logits, dim=-1)
    logprobs = torch.neg(torch.nn.functional.cross_entropy(logits, labels.reshape(-1), reduction="none"))
    d_hidden, d_weight = torch.autograd.grad((entropy, logprobs), (h, w), (g_entropy.to(compute_dtype), g_logprobs.to(compute_dtype)))
    return logprobs.detach(), entropy.detach(), d_hidden.reshape(hidden.shape), d_weight


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, compute_dtype=torch.float32):
    """log_softmax(logits)[label], with an explicit upcast (CPU log_softmax does not upcast bf16)."""
    z = logits.to(compute_dtype)
    lp = torch.log_softmax(z, dim=-1)
    return torch.gather(lp, -1, labels.long().unsqueeze(-1)).squeeze(-1)


def entropy_from_logits(logits: torch.Tensor, compute_dtype=torch.float32):
    """logsumexp(z) - sum(softmax(z) * z)."""
    z = logits.to(compute_dtype)
    pd = torch.softmax(z, dim=-1)
    return torch.logsumexp(z, dim=-1) - torch.sum(pd * z, dim=-1)


def sum_pi_squared_from_logits(logits: torch.Tensor, compute_dtype=torch.float32):
    """sum_v softmax(z)_v^2, stated as in the reference: exp(logsumexp(2 z) - 2 logsumexp(z))."""
    z = logits.to(compute_dtype)
    return torch.exp(torch.logsumexp(2.0 * z, dim=-1) - 2.0 * torch.logsumexp(z, dim=-1))


def logits_backward(
    logits: torch.Tensor,
    labels: Optional[torch.Tensor],
    dlogprobs: Optional[torch.Tensor],
    dentropy: Optional[torch.Tensor],
    compute_dtype=torch.float32,
):
    """d_logits of ``sum(dlogprobs * logprobs) + sum(dentropy * entropy)`` w.r.t. the logits."""
    z = logits.to(compute_dtype)
    p = torch.softmax(z, dim=-1)
    dz = torch.zeros_like(z)
    if dlogprobs is not None:
        g = dlogprobs.to(compute_dtype).unsqueeze(-1)
        dz -= g * p
        dz.scatter_add_(-1, labels.long().unsqueeze(-1), g.expand(*labels.shape, 1).clone())
    if dentropy is not None:
        b = torch.sum(p * z, dim=-1, keepdim=True)
        dz -= dentropy.to(compute_dtype).unsqueeze(-1) * p * (z - b)
    return dz


# ----------------------------------------------------------------------------------------------
# consumer of the path's output: the PPO actor loss
# ----------------------------------------------------------------------------------------------


def masked_sum(values, mask, axis=None):
    valid = torch.where(mask.bool(), values, torch.zeros((), dtype=values.dtype, device=values.device))
    return (valid * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None):
    return masked_sum(values, mask, axis) / (mask.sum(axis=axis) + 1e-8)


def agg_loss(
    loss_mat,
    loss_mask,
    loss_agg_mode: str,
    dp_size: int = 1,
    batch_num_tokens=None,
    global_batch_size=None,
    loss_scale_factor=None,
):
    if loss_agg_mode == "token-mean":
        if batch_num_tokens is None:
            if dp_size > 1:
                raise ValueError("(global) batch_num_tokens is required when dp_size > 1")
            batch_num_tokens = loss_mask.sum()
        return masked_sum(loss_mat, loss_mask) / batch_num_tokens * dp_size
    if loss_agg_mode == "token-sum":
        return masked_sum(loss_mat, loss_mask) * dp_size
    if loss_agg_mode in ("seq-mean-token-sum", "seq-mean-token-sum-norm"):
        seq_losses = torch.sum(loss_mat * loss_mask, dim=-1)
        seq_mask = (torch.sum(loss_mask, dim=-1) > 0).float()
        if global_batch_size is None:
            if dp_size > 1:
                raise ValueError("global_batch_size is required when dp_size > 1")
            global_batch_size = seq_mask.sum()
        loss = masked_sum(seq_losses, seq_mask) / global_batch_size * dp_size
        if loss_agg_mode == "seq-mean-token-sum-norm":
            loss = loss / (loss_mask.shape[-1] if loss_scale_factor is None else loss_scale_factor)
        return loss
    if loss_agg_mode == "seq-mean-token-mean":
        cnt = torch.sum(loss_mask, dim=-1)
        seq_losses = torch.sum(loss_mat * loss_mask, dim=-1) / (cnt + 1e-8)
        seq_mask = (cnt > 0).float()
        if global_batch_size is None:
            if dp_size > 1:
                raise ValueError("global_batch_size is required when dp_size > 1")
            global_batch_size = seq_mask.sum()
        return masked_sum(seq_losses, seq_mask) / global_batch_size * dp_size
    raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")


def policy_loss_vanilla(
    old_log_prob,
    log_prob,
    advantages,
    response_mask,
    loss_agg_mode: str = "token-mean",
    clip_ratio: float = 0.2,
    clip_ratio_low: Optional[float] = None,
    clip_ratio_high: Optional[float] = None,
    clip_ratio_c: float = 3.0,
    rollout_is_weights=None,
    **global_batch_info,
):
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    assert clip_ratio_c > 1.0
    nkl = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(nkl)
    ppo_kl = masked_mean(-nkl, response_mask)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - lo, 1 + hi)
    lc1 = torch.maximum(l1, l2)
    clipfrac = masked_mean(torch.gt(l2, l1).float(), response_mask)
    l3 = -advantages * clip_ratio_c
    lc2 = torch.min(l3, lc1)
    clipfrac_lower = masked_mean(torch.gt(lc1, l3) * (advantages < 0).float(), response_mask)
    losses = torch.where(advantages < 0, lc2, lc1)
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    loss = agg_loss(losses, response_mask, loss_agg_mode, **global_batch_info)
    metrics = {
        "actor/pg_clipfrac": clipfrac.detach().item(),
        "actor/ppo_kl": ppo_kl.detach().item(),
        "actor/pg_clipfrac_lower": clipfrac_lower.detach().item(),
    }
    return loss, metrics


def kl_penalty(logprob, ref_logprob, kl_penalty_type: str):
    """verl/trainer/ppo/core_algos.py:2188-2251: the k1 / abs / k2 / k3 estimators of KL(pi || pi_ref) per token; a
    trailing "+" keeps the estimator's value and gives it the gradient of k2 (straight through), k2 itself unchanged."""
    base = kl_penalty_type[:-1] if kl_penalty_type.endswith("+") else kl_penalty_type
    if base in ("kl", "k1"):
        fwd = logprob - ref_logprob
    elif base == "abs":
        fwd = (logprob - ref_logprob).abs()
    elif base in ("mse", "k2"):
        fwd = 0.5 * (logprob - ref_logprob).square()
    elif base in ("low_var_kl", "k3"):
        kl = torch.clamp(ref_logprob - logprob, min=-20, max=20)
        fwd = torch.clamp(torch.exp(kl) - kl - 1, min=-10, max=10)
    else:
        raise NotImplementedError
    if not kl_penalty_type.endswith("+") or kl_penalty_type in ("mse", "k2"):
        return fwd
    bwd = 0.5 * (logprob - ref_logprob).square()
    return bwd - bwd.detach() + fwd.detach()


def ppo_actor_loss(
    log_prob,
    entropy,
    old_log_prob,
    advantages,
    response_mask,
    clip_ratio: float = 0.2,
    entropy_coeff: float = 0.0,
    loss_agg_mode: str = "token-mean",
    clip_ratio_c: float = 3.0,
    rollout_is_weights=None,
    ref_log_prob=None,
    kl_loss_type: str = "low_var_kl",
    kl_loss_coef: float = 0.001,
    **global_batch_info,
):
    """policy loss - entropy_coeff * agg(entropy) [+ kl_loss_coef * agg(kl_penalty)]: the scalar the actor
    back-propagates (verl/workers/utils/losses.py:109-153; every term aggregated with the same mode and global
    batch info; the KL term is the reference's use_kl_loss branch, taken here when ref_log_prob is given)."""
    pg, metrics = policy_loss_vanilla(
        old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, clip_ratio, clip_ratio_c=clip_ratio_c,
        rollout_is_weights=rollout_is_weights, **global_batch_info,
    )  # fmt: skip
    loss = pg
    if entropy is not None:
        ent = agg_loss(entropy, response_mask, loss_agg_mode, **global_batch_info)
        loss = loss - entropy_coeff * ent
        metrics["actor/entropy_loss"] = ent.detach().item()
    if ref_log_prob is not None:
        kld = kl_penalty(log_prob, ref_log_prob, kl_loss_type)
        kl = agg_loss(kld, response_mask, loss_agg_mode, **global_batch_info)
        loss = loss + kl * kl_loss_coef
        metrics["kl_loss"] = kl.detach().item()
        metrics["kl_coef"] = kl_loss_coef
    metrics["actor/pg_loss"] = pg.detach().item()
    return loss, metrics


def no_padding_2_padding(values, prompt_lens, response_lens, max_response_len: Optional[int] = None):
    """verl/workers/utils/padding.py:97-141: the response slice of a packed per-token model output.  Sequence r
    occupies values[E_{r-1} : E_r], E_r = cumsum(prompt_lens + response_lens); its response part, left-shifted by one
    token (the output at position i predicts token i + 1), is values[E_r - R_r - 1 : E_r - 1], right-padded with zeros
    to max_response_len and stacked to [batch, max_response_len]."""
    prompt_lens = torch.as_tensor(prompt_lens)
    response_lens = torch.as_tensor(response_lens)
    if max_response_len is None:
        max_response_len = int(response_lens.max().item())
    offsets = (prompt_lens + response_lens).cumsum(dim=0)
    assert offsets[-1].item() == values.shape[0]
    assert not prompt_lens.eq(0).any(), f"seq_offset - resp_len - 1 assumes prompt_len > 0. Got {prompt_lens}"
    rows = []
    for resp_len, end in zip(response_lens.tolist(), offsets.tolist()):
        rows.append(torch.nn.functional.pad(values[end - resp_len - 1 : end - 1], (0, max_response_len - resp_len)))
    return torch.stack(rows, dim=0)


def padded_vocab_known_answer(V: int):
    """Closed form of the reference's padded-vocab regression: one logit +3 and V-1 logits -15.
    Returns (logprob of label 0, entropy) in double precision."""
    z0, z1, n1 = 3.0, -15.0, V - 1
    lse = z0 + math.log1p(n1 * math.exp(z1 - z0))
    p0 = math.exp(z0 - lse)
    p1 = math.exp(z1 - lse)
    return z0 - lse, lse - (p0 * z0 + n1 * p1 * z1)
