"""Fused PPO actor loss kernel against the oracle's restatement of compute_policy_loss_vanilla + agg_loss +
entropy bonus (verl/trainer/ppo/core_algos.py:1140-1206,1286-1376; verl/workers/utils/losses.py:57-140)."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(B, L, seed, spread=0.05):
    g = torch.Generator().manual_seed(seed)
    lp = -torch.rand(B, L, generator=g) * 3
    old = lp + torch.randn(B, L, generator=g) * spread
    adv = torch.randn(B, 1, generator=g).expand(B, L).contiguous()
    ent = torch.rand(B, L, generator=g) * 5
    valid = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None, :] < valid[:, None]).float()
    return [t.to(DEV) for t in (lp, ent, old, adv, mask)]


@pytest.mark.parametrize("spread", [0.05, 0.6, 3.0])  # 3.0 drives ratios into clip, dual-clip and the +-20 clamp
@pytest.mark.parametrize("with_entropy", [True, False])
def test_matches_oracle(spread, with_entropy):
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp, ent, old, adv, mask = _case(16, 257, seed=int(spread * 100), spread=spread)
    old = old + (torch.rand_like(old) < 0.01).float() * 25.0  # a few beyond the log-ratio clamp
    lp1 = lp.clone().requires_grad_(True)
    ent1 = ent.clone().requires_grad_(True) if with_entropy else None
    loss, met = fused_ppo_loss(lp1, ent1, old, adv, mask, clip_ratio=0.2, clip_ratio_c=3.0, entropy_coeff=1e-3)
    (loss * 1.7).backward()
    lp2 = lp.clone().requires_grad_(True)
    ent2 = ent.clone().requires_grad_(True) if with_entropy else None
    rloss, rmet = O.ppo_actor_loss(lp2, ent2, old, adv, mask, clip_ratio=0.2, entropy_coeff=1e-3)
    (rloss * 1.7).backward()
    torch.testing.assert_close(loss, rloss, atol=1e-6, rtol=1e-5)
    for k, v in met.items():
        assert v.item() == pytest.approx(rmet[k], rel=1e-5, abs=1e-6), k
    torch.testing.assert_close(lp1.grad, lp2.grad, atol=1e-8, rtol=1e-5)
    if with_entropy:
        torch.testing.assert_close(ent1.grad, ent2.grad, atol=1e-9, rtol=1e-5)
        assert (ent1.grad[mask == 0] == 0).all()
    assert (lp1.grad[mask == 0] == 0).all()


def test_global_batch_scaling_and_errors():
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp, ent, old, adv, mask = _case(4, 64, seed=3)
    loss, _ = fused_ppo_loss(lp, ent, old, adv, mask, entropy_coeff=0.01, dp_size=4, batch_num_tokens=1000)
    pg, _ = O.policy_loss_vanilla(old, lp, adv, mask, dp_size=4, batch_num_tokens=1000)
    want = pg - 0.01 * O.agg_loss(ent, mask, "token-mean", dp_size=4, batch_num_tokens=1000)
    torch.testing.assert_close(loss, want, atol=1e-6, rtol=1e-5)
    with pytest.raises(ValueError):
        fused_ppo_loss(lp, ent, old, adv, mask, dp_size=2)
    with pytest.raises(ValueError, match="global_batch_size is required"):
        fused_ppo_loss(lp, ent, old, adv, mask, dp_size=2, loss_agg_mode="seq-mean-token-sum")
    with pytest.raises(ValueError, match="Invalid loss_agg_mode"):  # core_algos.py:1203-1204
        fused_ppo_loss(lp, ent, old, adv, mask, loss_agg_mode="nope")
    # NaNs outside the mask do not leak (masked_sum semantics, verl/utils/torch_functional.py:273-291)
    lp_nan = lp.clone()
    lp_nan[mask == 0] = float("nan")
    loss_nan, _ = fused_ppo_loss(lp_nan, ent, old, adv, mask, entropy_coeff=0.01)
    loss_ok, _ = fused_ppo_loss(lp, ent, old, adv, mask, entropy_coeff=0.01)
    torch.testing.assert_close(loss_nan, loss_ok)


AGG_CASES = [
    ("token-mean", {}),
    ("token-mean", dict(dp_size=4, batch_num_tokens=5000)),
    ("token-sum", {}),
    ("token-sum", dict(dp_size=2)),
    ("seq-mean-token-sum", {}),
    ("seq-mean-token-sum", dict(dp_size=2, global_batch_size=64)),
    ("seq-mean-token-sum-norm", {}),
    ("seq-mean-token-sum-norm", dict(loss_scale_factor=1000)),
    ("seq-mean-token-sum-norm", dict(dp_size=8, global_batch_size=128, loss_scale_factor=512)),
    ("seq-mean-token-mean", {}),
    ("seq-mean-token-mean", dict(dp_size=2, global_batch_size=40)),
]


@pytest.mark.parametrize("mode,info", AGG_CASES)
@pytest.mark.parametrize("B,L", [(16, 257), (3, 5000), (5000, 3), (1, 1)])
def test_every_aggregation_mode(mode, info, B, L):
    """agg_loss's five modes (verl/trainer/ppo/core_algos.py:1172-1204) with and without the global batch
    information, rows without any valid token included, rollout correction weights on the policy term."""
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp, ent, old, adv, mask = _case(B, L, seed=B + L, spread=0.6)
    if B > 2:
        mask[1] = 0  # a fully masked sequence: left out of every sequence mean
    isw = torch.rand(B, L, device=DEV) * 2
    lp1, ent1 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    loss, met = fused_ppo_loss(lp1, ent1, old, adv, mask.bool(), entropy_coeff=1e-2, loss_agg_mode=mode,
                               rollout_is_weights=isw, **info)  # fmt: skip
    loss.backward()
    lp2, ent2 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    rloss, rmet = O.ppo_actor_loss(lp2, ent2, old, adv, mask, entropy_coeff=1e-2, loss_agg_mode=mode,
                                   rollout_is_weights=isw, **info)  # fmt: skip
    rloss.backward()
    torch.testing.assert_close(loss, rloss, atol=1e-6, rtol=2e-5)
    for k, v in met.items():
        assert v.item() == pytest.approx(rmet[k], rel=2e-5, abs=1e-6), k
    scale = max(lp2.grad.abs().max().item(), 1e-30)
    torch.testing.assert_close(lp1.grad, lp2.grad, atol=1e-6 * scale, rtol=1e-5)
    torch.testing.assert_close(ent1.grad, ent2.grad, atol=1e-6 * max(ent2.grad.abs().max().item(), 1e-30), rtol=1e-5)
    assert (lp1.grad[mask == 0] == 0).all() and (ent1.grad[mask == 0] == 0).all()
    # bit-identical on a second call (fixed reduction order)
    loss_b, _ = fused_ppo_loss(lp, ent, old, adv, mask, entropy_coeff=1e-2, loss_agg_mode=mode,
                               rollout_is_weights=isw, **info)  # fmt: skip
    assert loss_b.item() == loss.item()


def test_flat_token_list_equals_rows_in_token_modes():
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp, ent, old, adv, mask = _case(7, 300, seed=11)
    for mode in ("token-mean", "token-sum"):
        a, _ = fused_ppo_loss(lp, ent, old, adv, mask, entropy_coeff=1e-3, loss_agg_mode=mode)
        b, _ = fused_ppo_loss(lp.reshape(-1), ent.reshape(-1), old.reshape(-1), adv.reshape(-1), mask.reshape(-1),
                              entropy_coeff=1e-3, loss_agg_mode=mode)  # fmt: skip
        torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("kl_type", ["kl", "abs", "mse", "low_var_kl", "k1+", "abs+", "k2+", "k3+", "low_var_kl+"])
@pytest.mark.parametrize("mode", ["token-mean", "seq-mean-token-mean"])
def test_kl_penalty_term(kl_type, mode):
    """ppo_loss's use_kl_loss branch (verl/workers/utils/losses.py:142-153) with every estimator of kl_penalty
    (verl/trainer/ppo/core_algos.py:2188-2251), the oracle evaluated in fp64."""
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp, ent, old, adv, mask = _case(16, 257, seed=21, spread=0.3)
    g = torch.Generator().manual_seed(22)
    ref = lp + (torch.randn(16, 257, generator=g) * 0.2).to(DEV)
    ref[0, :4] = lp[0, :4] + torch.tensor([25.0, -25.0, 3.0, 0.0], device=DEV)  # both clamps of k3, and equality
    lp1, ent1 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    loss, met = fused_ppo_loss(lp1, ent1, old, adv, mask, entropy_coeff=1e-2, loss_agg_mode=mode, ref_log_prob=ref,
                               kl_loss_type=kl_type, kl_loss_coef=0.05)  # fmt: skip
    loss.backward()
    d = [t.double() for t in (lp, ent, old, adv, mask, ref)]
    lp2, ent2 = d[0].clone().requires_grad_(True), d[1].clone().requires_grad_(True)
    rloss, rmet = O.ppo_actor_loss(lp2, ent2, d[2], d[3], d[4], entropy_coeff=1e-2, loss_agg_mode=mode,
                                   ref_log_prob=d[5], kl_loss_type=kl_type, kl_loss_coef=0.05)  # fmt: skip
    rloss.backward()
    torch.testing.assert_close(loss.double(), rloss, atol=1e-6, rtol=2e-5)
    assert met["kl_coef"] == 0.05
    assert met["kl_loss"].item() == pytest.approx(rmet["kl_loss"], rel=2e-5, abs=1e-7)
    scale = lp2.grad.abs().max().item()
    torch.testing.assert_close(lp1.grad.double(), lp2.grad, atol=2e-6 * scale, rtol=2e-5)
    torch.testing.assert_close(ent1.grad.double(), ent2.grad, atol=1e-9, rtol=1e-5)
    with pytest.raises(NotImplementedError):
        fused_ppo_loss(lp, ent, old, adv, mask, ref_log_prob=ref, kl_loss_type="full")


@pytest.mark.parametrize("mode,info", AGG_CASES)
def test_agg_loss_and_policy_loss_under_the_reference_names(mode, info):
    """verl_amd.trainer.ppo.core_algos.agg_loss / compute_policy_loss_vanilla: the reference's signatures
    (verl/trainer/ppo/core_algos.py:1140-1206, :1286-1376), values and gradients against the oracle."""
    from types import SimpleNamespace

    from verl_amd.trainer.ppo.core_algos import agg_loss, compute_policy_loss_vanilla

    lp, ent, old, adv, mask = _case(9, 700, seed=31, spread=0.6)
    mask[4] = 0
    x1 = ent.clone().requires_grad_(True)
    got = agg_loss(x1, mask, mode, **info)
    (got * 3.0).backward()
    x2 = ent.clone().requires_grad_(True)
    want = O.agg_loss(x2, mask, mode, **info)
    (want * 3.0).backward()
    torch.testing.assert_close(got, want, atol=1e-6, rtol=2e-5)
    torch.testing.assert_close(x1.grad, x2.grad, atol=1e-6 * x2.grad.abs().max().item(), rtol=1e-5)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.1, clip_ratio_high=0.3, global_batch_info=info,
                          get=lambda k, dflt=None: {"clip_ratio_c": 2.5}.get(k, dflt))  # fmt: skip
    lp1 = lp.clone().requires_grad_(True)
    pg, pm = compute_policy_loss_vanilla(old, lp1, adv, mask, mode, cfg)
    pg.backward()
    lp2 = lp.clone().requires_grad_(True)
    rpg, rpm = O.policy_loss_vanilla(old, lp2, adv, mask, mode, 0.2, 0.1, 0.3, 2.5, **info)
    rpg.backward()
    torch.testing.assert_close(pg, rpg, atol=1e-6, rtol=2e-5)
    assert set(pm) == set(rpm) and all(isinstance(v, float) for v in pm.values())
    for k in pm:
        assert pm[k] == pytest.approx(rpm[k], rel=2e-5, abs=1e-6), k
    torch.testing.assert_close(lp1.grad, lp2.grad, atol=1e-6 * lp2.grad.abs().max().item(), rtol=1e-5)


def test_agg_loss_errors_like_the_reference():
    from verl_amd.trainer.ppo.core_algos import agg_loss

    lp, ent, old, adv, mask = _case(2, 8, seed=1)
    with pytest.raises(ValueError, match="Invalid loss_agg_mode"):
        agg_loss(ent, mask, "nope")
    with pytest.raises(ValueError, match="batch_num_tokens is required"):
        agg_loss(ent, mask, "token-mean", dp_size=2)
    with pytest.raises(ValueError, match="global_batch_size is required"):
        agg_loss(ent, mask, "seq-mean-token-mean", dp_size=2)
    # the reference's own known answers (tests/trainer/ppo/test_loss_aggregation_on_cpu.py:23-30)
    loss_mat = torch.tensor([[1.0, 2.0, 30.0], [4.0, 50.0, 6.0]], device=DEV)
    loss_mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 0.0, 1.0]], device=DEV)
    assert agg_loss(loss_mat, loss_mask, "token-sum", dp_size=4).item() == pytest.approx((1 + 2 + 4 + 6) * 4)
    assert agg_loss(loss_mat, loss_mask, "seq-mean-token-mean").item() == pytest.approx((1.5 + 5) / 2)


def test_actor_step_fused_end_to_end():
    """fused head -> fused loss -> fused backward, against the all-oracle pipeline (config-5 family, reduced)."""
    from verl_amd import linear_cross_entropy
    from verl_amd.workers.utils.losses import fused_ppo_loss

    H, V, nseq, L = 1024, 32000, 8, 128
    T = nseq * L
    g = torch.Generator(device=DEV).manual_seed(7)
    h = torch.randn(T, H, device=DEV, generator=g).bfloat16()
    w = (torch.randn(V, H, device=DEV, generator=g) * 0.02).bfloat16()
    y = torch.randint(0, V, (T,), device=DEV, generator=g)
    valid = torch.randint(8, L + 1, (nseq,), device=DEV, generator=g)
    mask = (torch.arange(L, device=DEV)[None, :] < valid[:, None]).float()
    adv = torch.randn(nseq, 1, device=DEV, generator=g).expand(nseq, L).contiguous()
    noise = torch.randn(nseq, L, device=DEV, generator=g) * 0.05
    hh = h.clone().requires_grad_(True)
    ww = w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(hh, ww, y, 1.0, "none")
    old = lp.detach().view(nseq, L) + noise
    loss, _ = fused_ppo_loss(lp.view(nseq, L), ent.view(nseq, L), old, adv, mask, entropy_coeff=1e-3)
    loss.backward()
    h2 = h.clone().requires_grad_(True)
    w2 = w.clone().requires_grad_(True)
    z = h2.float() @ w2.float().t()
    rlp = torch.log_softmax(z, -1).gather(-1, y[:, None]).squeeze(-1)
    rent = torch.logsumexp(z, -1) - (torch.softmax(z, -1) * z).sum(-1)
    rloss, _ = O.ppo_actor_loss(rlp.view(nseq, L), rent.view(nseq, L), old, adv, mask, entropy_coeff=1e-3)
    rloss.backward()
    torch.testing.assert_close(loss, rloss, atol=1e-4, rtol=1e-4)
    assert (hh.grad.float() - h2.grad).abs().max() <= 2e-2 * h2.grad.abs().max()
    assert (ww.grad.float() - w2.grad).abs().max() <= 2e-2 * w2.grad.abs().max()


def _packed_case(prompt, resp, R, seed):
    g = torch.Generator().manual_seed(seed)
    B, total = len(prompt), int(sum(prompt) + sum(resp))
    lp = -torch.rand(total, generator=g) * 3
    ent = torch.rand(total, generator=g) * 5
    old = -torch.rand(B, R, generator=g) * 3
    adv = torch.randn(B, 1, generator=g).expand(B, R).contiguous()
    ref = -torch.rand(B, R, generator=g) * 3
    mask = (torch.arange(R)[None, :] < torch.tensor(resp)[:, None]).float()
    mask = mask * (torch.rand(B, R, generator=g) > 0.1).float()  # holes inside the responses too
    return [t.to(DEV) for t in (lp, ent, old, adv, ref, mask)]


@pytest.mark.parametrize("mode", ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean"])
@pytest.mark.parametrize("with_kl", [False, True])
def test_packed_outputs_response_slice_inside_the_kernel(mode, with_kl):
    """fused_ppo_loss_packed against oracle slice (no_padding_2_padding, verl/workers/utils/padding.py:97-141) + oracle
    loss: ragged prompts and responses, response lengths 0 and 1, a row as long as the padded width, holes in the mask;
    the gradients come back in packed order and are exactly zero where no response position maps to."""
    from verl_amd.workers.utils.losses import fused_ppo_loss_packed

    prompt, resp = [3, 1, 7, 2, 1, 4, 260], [5, 1, 0, 9, 300, 2, 17]
    R = 300
    lp, ent, old, adv, ref, mask = _packed_case(prompt, resp, R, seed=5)
    P, Rl = torch.tensor(prompt, device=DEV), torch.tensor(resp, device=DEV)
    kw = dict(clip_ratio=0.2, entropy_coeff=1e-3, loss_agg_mode=mode)
    if with_kl:
        kw.update(ref_log_prob=ref, kl_loss_type="low_var_kl", kl_loss_coef=0.01)
    lp1, ent1 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    loss, met = fused_ppo_loss_packed(lp1, ent1, P, Rl, old, adv, mask, clip_ratio_c=3.0, **kw)
    (loss * 1.3).backward()
    lp2, ent2 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    rloss, rmet = O.ppo_actor_loss(O.no_padding_2_padding(lp2, prompt, resp, R), O.no_padding_2_padding(ent2, prompt, resp, R),
                                   old, adv, mask, **kw)
    (rloss * 1.3).backward()
    torch.testing.assert_close(loss, rloss, atol=1e-6, rtol=1e-5)
    for k, v in met.items():
        if k != "kl_coef":
            assert v.item() == pytest.approx(rmet[k], rel=1e-5, abs=1e-6), k
    assert lp1.grad.shape == lp.shape and ent1.grad.shape == ent.shape
    torch.testing.assert_close(lp1.grad, lp2.grad, atol=1e-8, rtol=1e-5)
    torch.testing.assert_close(ent1.grad, ent2.grad, atol=1e-9, rtol=1e-5)
    assert ((lp2.grad == 0) <= (lp1.grad == 0)).all()  # exact zeros wherever the oracle's gradient is zero
    # the same numbers as the padded entry point on the oracle's slice
    from verl_amd.workers.utils.losses import fused_ppo_loss

    loss_p, _ = fused_ppo_loss(O.no_padding_2_padding(lp, prompt, resp, R), O.no_padding_2_padding(ent, prompt, resp, R), old, adv, mask,
                               clip_ratio_c=3.0, **kw)
    torch.testing.assert_close(loss.detach(), loss_p, atol=0, rtol=0)


def test_packed_outputs_reference_assertions():
    from verl_amd.workers.utils.losses import fused_ppo_loss_packed

    prompt, resp, R = [2, 1, 3], [3, 1, 0], 4
    lp, ent, old, adv, ref, mask = _packed_case(prompt, resp, R, seed=6)
    P, Rl = torch.tensor(prompt, device=DEV), torch.tensor(resp, device=DEV)
    with pytest.raises(AssertionError, match="prompt_len > 0"):  # verl/workers/utils/padding.py:128
        fused_ppo_loss_packed(lp, ent, torch.tensor([2, 0, 4], device=DEV), Rl, old, adv, mask)
    with pytest.raises(AssertionError):  # lengths that do not add up to total_nnz (:127)
        fused_ppo_loss_packed(lp[:-1], ent[:-1], P, Rl, old, adv, mask)
    with pytest.raises(AssertionError, match="longer than max_response_len"):
        fused_ppo_loss_packed(lp, ent, P, Rl, old[:, :2], adv[:, :2], mask[:, :2])
    loss, _ = fused_ppo_loss_packed(lp, None, P, Rl, old, adv, mask)  # entropy is optional as in fused_ppo_loss
    assert torch.isfinite(loss)


class _ActorConfig:
    """The fields of the reference's ActorConfig that ppo_loss reads (verl/workers/utils/losses.py:57-155)."""

    def __init__(self, **kw):
        self.clip_ratio, self.clip_ratio_low, self.clip_ratio_high, self.clip_ratio_c = 0.2, None, None, 3.0
        self.entropy_coeff, self.loss_agg_mode, self.loss_scale_factor = 1e-3, "token-mean", None
        self.use_kl_loss, self.kl_loss_coef, self.kl_loss_type = False, 0.01, "low_var_kl"
        self.policy_loss = {"loss_mode": "vanilla"}
        self.global_batch_info = {}
        self.__dict__.update(kw)


def _jagged(values, lens):
    offsets = torch.cat([torch.zeros(1, dtype=torch.int64), torch.tensor(lens).cumsum(0)]).to(values.device)
    return torch.nested.nested_tensor_from_jagged(values, offsets=offsets)


@pytest.mark.parametrize("nested", [True, False])
@pytest.mark.parametrize("globals_set", [False, True])
def test_ppo_loss_entry_with_the_reference_signature(nested, globals_set):
    """ppo_loss(config, model_output, data) on a nested (no-padding) batch and on a padded batch with attention_mask:
    loss, gradients in packed order and every metric against the oracle's slice + loss; metric aggregation kinds as
    verl/workers/utils/losses.py:71-84,124-126 (pg statistics MEAN; losses SUM once a global normaliser is set)."""
    from verl_amd.utils.metric import AggregationType, Metric
    from verl_amd.workers.utils.losses import ppo_loss

    prompt, resp = [3, 1, 7, 2, 5], [5, 1, 12, 9, 2]
    R = 12 if nested else 16
    lp, ent, old, adv, ref, mask = _packed_case(prompt, resp, R, seed=11)
    B, total = len(prompt), lp.numel()
    ids = torch.arange(total, device=DEV)
    data = {"response_mask": mask, "old_log_probs": old, "advantages": adv, "ref_log_prob": ref,
            "dp_size": 2 if globals_set else 1, "batch_num_tokens": 77 if globals_set else None, "global_batch_size": None}
    if nested:
        data["prompts"] = _jagged(torch.arange(sum(prompt), device=DEV), prompt)
        data["responses"] = _jagged(torch.arange(sum(resp), device=DEV), resp)
        model_output = {"log_probs": _jagged(lp, [p + r for p, r in zip(prompt, resp)]), "entropy": None}
    else:
        Pw = 8
        data["prompts"] = torch.zeros(B, Pw, dtype=torch.long, device=DEV)
        data["responses"] = torch.zeros(B, R, dtype=torch.long, device=DEV)
        am = torch.zeros(B, Pw + R, dtype=torch.long, device=DEV)
        for b in range(B):
            am[b, Pw - prompt[b] : Pw + resp[b]] = 1  # left-padded prompts, right-padded responses
        data["attention_mask"] = am
        model_output = {"log_probs": None, "entropy": None}
    cfg = _ActorConfig(use_kl_loss=True, loss_agg_mode="token-mean")
    lp1, ent1 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    if nested:
        model_output["log_probs"] = _jagged(lp1, [p + r for p, r in zip(prompt, resp)])
        model_output["entropy"] = _jagged(ent1, [p + r for p, r in zip(prompt, resp)])
    else:
        model_output["log_probs"], model_output["entropy"] = lp1, ent1
    loss, metrics = ppo_loss(cfg, model_output, data)
    loss.backward()
    info = dict(dp_size=data["dp_size"], batch_num_tokens=data["batch_num_tokens"], global_batch_size=None, loss_scale_factor=None)
    assert cfg.global_batch_info == info  # left on the config as the reference does (:70-73)
    lp2, ent2 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    rloss, rmet = O.ppo_actor_loss(O.no_padding_2_padding(lp2, prompt, resp, R), O.no_padding_2_padding(ent2, prompt, resp, R), old, adv, mask,
                                   clip_ratio=0.2, entropy_coeff=1e-3, loss_agg_mode="token-mean", ref_log_prob=ref,
                                   kl_loss_type="low_var_kl", kl_loss_coef=0.01, **info)
    rloss.backward()
    torch.testing.assert_close(loss, rloss, atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(lp1.grad, lp2.grad, atol=1e-8, rtol=1e-5)
    torch.testing.assert_close(ent1.grad, ent2.grad, atol=1e-9, rtol=1e-5)
    want = AggregationType.SUM if globals_set else AggregationType.MEAN
    assert set(metrics) == {"actor/pg_clipfrac", "actor/ppo_kl", "actor/pg_clipfrac_lower", "actor/pg_loss", "actor/entropy_loss", "kl_loss", "kl_coef"}
    for k in ("actor/pg_clipfrac", "actor/ppo_kl", "actor/pg_clipfrac_lower"):
        assert isinstance(metrics[k], Metric) and metrics[k].aggregation == AggregationType.MEAN
    for k in ("actor/pg_loss", "actor/entropy_loss", "kl_loss"):
        assert metrics[k].aggregation == want
    for k, v in metrics.items():
        if k != "kl_coef":
            assert v.aggregate() == pytest.approx(rmet[k], rel=1e-5, abs=1e-6), k
    assert metrics["kl_coef"] == 0.01


@pytest.mark.parametrize("fields", ["jagged", "padded-wider", "padded-narrower"])
def test_ppo_loss_honours_max_response_len(fields):
    """verl/workers/utils/padding.py:112-118: on a nested batch the padded width of the response slice is the non-tensor
    entry max_response_len when it is given, else the longest response.  Every field of the batch is brought to exactly
    that width, whatever width it arrives in (jagged, padded wider, padded to the longest row only); a width shorter
    than the longest response is an error."""
    from verl_amd.workers.utils.losses import ppo_loss

    prompt, resp = [3, 1, 7, 2, 5], [5, 1, 12, 9, 2]
    R = 15  # max_response_len, larger than the longest response (12)
    lp, ent, old, adv, ref, mask = _packed_case(prompt, resp, R, seed=21)
    cols = torch.arange(R, device=DEV)[None, :] < torch.tensor(resp, device=DEV)[:, None]

    def field(t):
        if fields == "jagged":
            return _jagged(t[cols], resp)
        if fields == "padded-wider":
            return torch.nn.functional.pad(t, (0, 4), value=7.0)  # garbage beyond the width must never be read
        return t[:, :12].contiguous()

    data = {"prompts": _jagged(torch.arange(sum(prompt), device=DEV), prompt), "responses": _jagged(torch.arange(sum(resp), device=DEV), resp),
            "response_mask": field(mask), "old_log_probs": field(old), "advantages": field(adv), "ref_log_prob": field(ref),
            "max_response_len": R, "dp_size": 1, "batch_num_tokens": None, "global_batch_size": None}
    cfg = _ActorConfig(use_kl_loss=True, loss_agg_mode="seq-mean-token-sum-norm", loss_scale_factor=None)
    lp1, ent1 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    lens = [p + r for p, r in zip(prompt, resp)]
    loss, metrics = ppo_loss(cfg, {"log_probs": _jagged(lp1, lens), "entropy": _jagged(ent1, lens)}, data)
    loss.backward()
    lp2, ent2 = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
    pad = lambda t: t * cols  # noqa: E731  (what the reference's to_padded_tensor leaves beyond a row's end: zeros)
    rloss, rmet = O.ppo_actor_loss(O.no_padding_2_padding(lp2, prompt, resp, R), O.no_padding_2_padding(ent2, prompt, resp, R), pad(old),
                                   pad(adv), pad(mask), clip_ratio=0.2, entropy_coeff=1e-3, loss_agg_mode="seq-mean-token-sum-norm",
                                   ref_log_prob=pad(ref), kl_loss_type="low_var_kl", kl_loss_coef=0.01, dp_size=1, batch_num_tokens=None,
                                   global_batch_size=None, loss_scale_factor=None)
    rloss.backward()
    # (seq-mean-token-sum-norm divides by the padded width: the result depends on max_response_len, which is the point)
    torch.testing.assert_close(loss, rloss, atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(lp1.grad, lp2.grad, atol=1e-8, rtol=1e-5)
    torch.testing.assert_close(ent1.grad, ent2.grad, atol=1e-9, rtol=1e-5)
    for k in ("actor/pg_loss", "actor/entropy_loss", "kl_loss", "actor/ppo_kl"):
        assert metrics[k].aggregate() == pytest.approx(rmet[k], rel=1e-5, abs=1e-6), k
    data["max_response_len"] = 11
    with pytest.raises(ValueError, match="shorter than the longest response"):
        ppo_loss(cfg, {"log_probs": _jagged(lp1, lens), "entropy": _jagged(ent1, lens)}, data)


def test_ppo_loss_entry_refuses_what_has_no_fused_kernel():
    from verl_amd.workers.utils.losses import ppo_loss

    prompt, resp, R = [2, 1], [3, 1], 3
    lp, ent, old, adv, ref, mask = _packed_case(prompt, resp, R, seed=12)
    data = {"prompts": _jagged(torch.arange(3, device=DEV), prompt), "responses": _jagged(torch.arange(4, device=DEV), resp),
            "response_mask": mask, "old_log_probs": old, "advantages": adv, "dp_size": 1, "batch_num_tokens": None, "global_batch_size": None}
    with pytest.raises(NotImplementedError, match="only 'vanilla'"):
        ppo_loss(_ActorConfig(policy_loss={"loss_mode": "gspo"}), {"log_probs": lp}, data)
    with pytest.raises(NotImplementedError, match="sampler-correction"):
        ppo_loss(_ActorConfig(), {"log_probs": lp, "sc_correction": lp}, data)
    loss, metrics = ppo_loss(_ActorConfig(), {"log_probs": lp}, data)  # no entropy, no KL: just the policy loss
    assert torch.isfinite(loss) and "actor/entropy_loss" not in metrics and "kl_loss" not in metrics


def test_deprecated_compute_policy_loss_name():
    """core_algos.py:1210-1282: positional cliprange arguments, a 4-tuple back, FutureWarning like the reference's decorator."""
    from verl_amd.trainer.ppo import core_algos as C

    lp, _, old, adv, mask = _case(6, 40, seed=21, spread=0.6)
    with pytest.warns(FutureWarning, match="compute_policy_loss_vanilla"):
        pg, clipfrac, kl, clipfrac_lower = C.compute_policy_loss(old, lp, adv, mask, 0.2, 0.1, 0.3, 2.5, "seq-mean-token-mean")
    r, m = O.policy_loss_vanilla(old, lp, adv, mask, "seq-mean-token-mean", 0.2, clip_ratio_low=0.1, clip_ratio_high=0.3, clip_ratio_c=2.5)
    torch.testing.assert_close(pg, r, atol=1e-6, rtol=1e-5)
    assert clipfrac.item() == pytest.approx(m["actor/pg_clipfrac"], rel=1e-5, abs=1e-7)
    assert kl.item() == pytest.approx(m["actor/ppo_kl"], rel=1e-5, abs=1e-7)
    assert clipfrac_lower.item() == pytest.approx(m["actor/pg_clipfrac_lower"], rel=1e-5, abs=1e-7)
    assert C.get_policy_loss_fn("vanilla") is C.compute_policy_loss_vanilla
    with pytest.raises(ValueError, match="Unsupported loss mode: gpg"):
        C.get_policy_loss_fn("gpg")
