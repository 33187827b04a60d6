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


def test_kl_penalty_estimators_against_scalar_arithmetic():
    """verl/trainer/ppo/core_algos.py:2188-2251, pinned by the definitions evaluated with math.exp on scalars, the
    textbook facts about the estimators (k3 >= 0 with equality at equal log-probs, k3 ~ k2 for small differences,
    E_pi[k1] = E_pi[k3] = KL on a small categorical distribution) and autograd for the straight-through variants."""
    import math

    lp = torch.tensor([-1.0, -0.5, -2.0, -0.7, -30.0, 5.0], dtype=torch.float64)
    ref = torch.tensor([-1.5, -0.5, -1.0, -0.71, 0.0, -30.0], dtype=torch.float64)
    for i in range(6):
        d = lp[i].item() - ref[i].item()
        q = min(max(-d, -20.0), 20.0)
        want = {"kl": d, "abs": abs(d), "mse": 0.5 * d * d, "low_var_kl": min(max(math.exp(q) - q - 1, -10.0), 10.0)}
        for name, alias in (("kl", "k1"), ("abs", "abs"), ("mse", "k2"), ("low_var_kl", "k3")):
            assert O.kl_penalty(lp, ref, name)[i].item() == pytest.approx(want[name], rel=1e-12, abs=1e-15)
            assert O.kl_penalty(lp, ref, alias)[i].item() == pytest.approx(want[name], rel=1e-12, abs=1e-15)
    k3 = O.kl_penalty(lp, ref, "k3")
    assert (k3 >= 0).all() and k3[1].item() == 0.0
    assert k3[3].item() == pytest.approx(0.5 * 0.01**2, rel=1e-2)  # k3 = d^2/2 + O(d^3)
    assert k3[4].item() == 10.0  # exp(20) - 20 - 1 clamped to 10
    assert k3[5].item() == 10.0  # exp(-20) + 20 - 1 = 19.0 clamped to 10
    # expectations over a categorical pi: sum_x pi(x) k1(x) = KL(pi || ref) = sum_x pi(x) k3(x)
    pi = torch.tensor([0.5, 0.3, 0.2], dtype=torch.float64)
    rf = torch.tensor([0.2, 0.5, 0.3], dtype=torch.float64)
    kl_true = (pi * (pi / rf).log()).sum().item()
    assert (pi * O.kl_penalty(pi.log(), rf.log(), "k1")).sum().item() == pytest.approx(kl_true, rel=1e-12)
    assert (pi * O.kl_penalty(pi.log(), rf.log(), "k3")).sum().item() == pytest.approx(kl_true, rel=1e-12)
    # straight-through: the value of the estimator, the gradient of k2 (= log_prob - ref_log_prob)
    for name in ("kl+", "abs+", "low_var_kl+", "k3+", "k2+", "mse+"):
        x = lp.clone().requires_grad_(True)
        v = O.kl_penalty(x, ref, name)
        torch.testing.assert_close(v.detach(), O.kl_penalty(lp, ref, name[:-1]))
        v.sum().backward()
        torch.testing.assert_close(x.grad, lp - ref)
    with pytest.raises(NotImplementedError):
        O.kl_penalty(lp, ref, "full")


def test_actor_loss_with_kl_term_is_the_sum_of_its_parts():
    g = torch.Generator().manual_seed(5)
    lp = -torch.rand(3, 7, generator=g)
    old = lp + 0.1 * torch.randn(3, 7, generator=g)
    ref = lp + 0.2 * torch.randn(3, 7, generator=g)
    adv = torch.randn(3, 7, generator=g)
    ent = torch.rand(3, 7, generator=g)
    mask = (torch.rand(3, 7, generator=g) < 0.7).float()
    for mode in ("token-mean", "seq-mean-token-mean"):
        loss, met = O.ppo_actor_loss(lp, ent, old, adv, mask, entropy_coeff=0.1, loss_agg_mode=mode, ref_log_prob=ref,
                                     kl_loss_type="low_var_kl", kl_loss_coef=0.3)  # fmt: skip
        pg, _ = O.policy_loss_vanilla(old, lp, adv, mask, mode)
        want = pg - 0.1 * O.agg_loss(ent, mask, mode) + 0.3 * O.agg_loss(O.kl_penalty(lp, ref, "k3"), mask, mode)
        torch.testing.assert_close(loss, want)
        assert met["kl_coef"] == 0.3 and met["kl_loss"] == pytest.approx(O.agg_loss(O.kl_penalty(lp, ref, "k3"), mask, mode).item())


def test_response_slice_of_packed_outputs_hand_written_batch():
    """no_padding_2_padding (verl/workers/utils/padding.py:97-141) on a packed batch written out by hand: three
    sequences with (prompt, response) lengths (2, 3), (1, 1), (3, 0); the packed per-token values are 100 * sequence +
    position.  The response part is left-shifted by one token: sequence 0 occupies packed[0:5] and its response slice
    is positions 1..3 (the outputs that PREDICT the three response tokens at positions 2..4)."""
    values = torch.tensor([0.0, 1, 2, 3, 4, 100, 101, 200, 201, 202])
    out = O.no_padding_2_padding(values, [2, 1, 3], [3, 1, 0], max_response_len=4)
    want = torch.tensor([[1.0, 2, 3, 0], [100, 0, 0, 0], [0, 0, 0, 0]])
    assert torch.equal(out, want)
    # default width = the longest response
    assert torch.equal(O.no_padding_2_padding(values, [2, 1, 3], [3, 1, 0]), want[:, :3])
    # the reference's two assertions
    with pytest.raises(AssertionError, match="prompt_len > 0"):
        O.no_padding_2_padding(values, [2, 0, 3], [3, 2, 0])
    with pytest.raises(AssertionError):
        O.no_padding_2_padding(values[:-1], [2, 1, 3], [3, 1, 0])
    # a slice never takes the last token's output of its sequence and never reaches into the previous sequence
    v = torch.arange(12.0)
    got = O.no_padding_2_padding(v, [1, 1], [5, 5])
    assert torch.equal(got, torch.tensor([[0.0, 1, 2, 3, 4], [6, 7, 8, 9, 10]]))
