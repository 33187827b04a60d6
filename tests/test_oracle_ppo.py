"""Pins the restated PPO-loss consumer (oracle/lce_oracle.py) with the reference's known answers
(tests/trainer/ppo/test_loss_aggregation_on_cpu.py:23-65, tests/utils/test_torch_functional.py:61-72)
and closed-form special cases of verl/trainer/ppo/core_algos.py:1336-1369."""

import math

import pytest
import torch

from oracle import lce_oracle as O


def test_token_sum_known_answer():
    loss_mat = torch.tensor([[1.0, 2.0, 30.0], [4.0, 50.0, 6.0]])
    loss_mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 0.0, 1.0]])
    assert O.agg_loss(loss_mat, loss_mask, "token-sum", dp_size=4).item() == pytest.approx((1 + 2 + 4 + 6) * 4)
    assert O.agg_loss(loss_mat, loss_mask, "token-mean").item() == pytest.approx((1 + 2 + 4 + 6) / 4)
    assert O.agg_loss(loss_mat, loss_mask, "seq-mean-token-sum").item() == pytest.approx((3 + 10) / 2)
    assert O.agg_loss(loss_mat, loss_mask, "seq-mean-token-mean").item() == pytest.approx((1.5 + 5) / 2)
    assert O.agg_loss(loss_mat, loss_mask, "seq-mean-token-sum-norm").item() == pytest.approx((3 + 10) / 2 / 3)
    with pytest.raises(ValueError):
        O.agg_loss(loss_mat, loss_mask, "nope")
    with pytest.raises(ValueError):
        O.agg_loss(loss_mat, loss_mask, "token-mean", dp_size=2)


@pytest.mark.parametrize("num_micro_batches", [1, 2, 4])
def test_token_sum_microbatch_invariant(num_micro_batches):
    loss_mat = torch.arange(1, 25, dtype=torch.float32).reshape(8, 3)
    loss_mask = torch.tensor([[1.0, 1.0, 0.0]] * 8)
    step = 8 // num_micro_batches
    acc = sum(O.agg_loss(loss_mat[i : i + step], loss_mask[i : i + step], "token-sum") for i in range(0, 8, step))
    torch.testing.assert_close(acc, O.agg_loss(loss_mat, loss_mask, "token-sum"))


def test_masked_mean_known_answers():
    v = torch.tensor([1.0, 2.0, 3.0, 4.0])
    m = torch.tensor([0.0, 1.0, 1.0, 0.0])
    assert O.masked_mean(v, m).item() == pytest.approx(2.5)
    v_nan_out = torch.tensor([float("nan"), 2.0, 3.0, float("nan")])
    assert O.masked_mean(v_nan_out, m).item() == pytest.approx(2.5)
    v_nan_in = torch.tensor([1.0, float("nan"), 3.0, 4.0])
    assert math.isnan(O.masked_mean(v_nan_in, m).item())


def test_policy_loss_special_cases():
    mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 1.0, 1.0]])
    adv = torch.tensor([[1.0, -2.0, 5.0], [0.5, 0.5, -1.0]])
    lp = torch.tensor([[-1.0, -2.0, -3.0], [-0.5, -0.1, -4.0]])
    # identical policies: ratio 1, loss = -masked-mean(A), no clipping, zero KL
    loss, met = O.policy_loss_vanilla(lp, lp, adv, mask)
    assert loss.item() == pytest.approx(-(1 - 2 + 0.5 + 0.5 - 1) / 5)
    assert met["actor/pg_clipfrac"] == 0 and met["actor/ppo_kl"] == pytest.approx(0.0, abs=1e-7)
    # ratio e^{0.5} > 1.2 with A>0: clipped at 1.2 (gradient zero there)
    one = torch.ones(1, 1)
    new = torch.full((1, 1), 0.5, requires_grad=True)
    loss, met = O.policy_loss_vanilla(torch.zeros(1, 1), new, 2 * one, one)
    assert loss.item() == pytest.approx(-2 * 1.2)
    loss.backward()
    assert new.grad.item() == 0.0 and met["actor/pg_clipfrac"] == pytest.approx(1.0)
    # ratio e^{-0.5} < 0.8 with A<0: clipped at 0.8
    loss, _ = O.policy_loss_vanilla(torch.zeros(1, 1), torch.full((1, 1), -0.5), -2 * one, one)
    assert loss.item() == pytest.approx(2 * 0.8)
    # dual clip: A<0 and ratio e^{2} > 3: loss = -A*3
    loss, met = O.policy_loss_vanilla(torch.zeros(1, 1), torch.full((1, 1), 2.0), -2 * one, one)
    assert loss.item() == pytest.approx(2 * 3.0) and met["actor/pg_clipfrac_lower"] == pytest.approx(1.0)
    # inside the clip range the gradient is -A*ratio/N
    new = torch.full((1, 2), 0.05, requires_grad=True)
    loss, _ = O.policy_loss_vanilla(torch.zeros(1, 2), new, torch.tensor([[1.0, -1.0]]), torch.ones(1, 2))
    loss.backward()
    torch.testing.assert_close(new.grad, torch.tensor([[-1.0, 1.0]]) * math.exp(0.05) / 2)
    # log-ratio clamp at +-20
    loss, _ = O.policy_loss_vanilla(torch.zeros(1, 1), torch.full((1, 1), 50.0), one, one)
    assert loss.item() == pytest.approx(-1.2)


def test_ppo_actor_loss_entropy_bonus():
    mask = torch.tensor([[1.0, 1.0, 0.0]])
    lp = torch.tensor([[-1.0, -2.0, -3.0]])
    ent = torch.tensor([[2.0, 4.0, 100.0]], requires_grad=True)
    adv = torch.ones(1, 3)
    loss, met = O.ppo_actor_loss(lp, ent, lp, adv, mask, entropy_coeff=1e-3)
    assert loss.item() == pytest.approx(-1.0 - 1e-3 * 3.0)
    loss.backward()
    torch.testing.assert_close(ent.grad, torch.tensor([[-5e-4, -5e-4, 0.0]]))
    assert met["actor/entropy_loss"] == pytest.approx(3.0)
