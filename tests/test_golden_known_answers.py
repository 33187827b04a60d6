"""tests/golden/lce_known_answers.json (closed forms at 40 digits, written by tests/golden/make_known_answers.py)
against the torch oracle, the C oracle and, on the GPU, the HIP kernels through the C ABI."""

import json
import os

import pytest
import torch

from oracle import lce_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "lce_known_answers.json")) as f:
    GOLD = json.load(f)


def _two_level_inputs(case, H=128, T=3, dtype=torch.float64, tau=1.0):
    """hidden = e_0, W[:, 0] = logits * tau: the logits are exactly (z0, z1, z1, ...)."""
    V = case["V"]
    w = torch.zeros(V, H, dtype=dtype)
    w[:, 0] = case["z1"] * tau
    w[0, 0] = case["z0"] * tau
    h = torch.zeros(T, H, dtype=dtype)
    h[:, 0] = 1.0
    return h, w, torch.zeros(T, dtype=torch.long)


@pytest.mark.parametrize("case", GOLD["two_level"], ids=lambda c: f"V{c['V']}_{c['z0']}_{c['z1']}")
def test_two_level_oracles(case):
    h, w, y = _two_level_inputs(case, tau=1.5)
    lp, ent = O.lce_forward(h, w, y, 1.5, compute_dtype=torch.float64)
    assert lp[0].item() == pytest.approx(float(case["logprob"]), rel=1e-9, abs=1e-13)
    assert ent[0].item() == pytest.approx(float(case["entropy"]), rel=1e-9, abs=1e-13)
    if case["V"] <= 5000:
        from oracle import c_oracle

        out = c_oracle.forward(h.float().numpy(), w.float().numpy(), y.numpy(), 1.5)
        clp, cent = out["logprob"], out["entropy"]
        assert float(clp[0]) == pytest.approx(float(case["logprob"]), rel=1e-5, abs=1e-6)
        assert float(cent[0]) == pytest.approx(float(case["entropy"]), rel=1e-5, abs=1e-6)


@pytest.mark.parametrize("case", GOLD["uniform"], ids=lambda c: f"V{c['V']}")
def test_uniform_oracles(case):
    V = case["V"]
    z = torch.full((2, V), 0.37, dtype=torch.float64)
    # (the oracle of the unfused twins computes in fp32, like the functions it restates)
    assert O.entropy_from_logits(z)[0].item() == pytest.approx(float(case["entropy"]), rel=2e-6)
    assert O.logprobs_from_logits(z, torch.tensor([0, V - 1]))[1].item() == pytest.approx(float(case["logprob"]), rel=2e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLD["two_level"], ids=lambda c: f"V{c['V']}_{c['z0']}_{c['z1']}")
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_two_level_kernels(case, dtype):
    """All values involved are exact in bf16 (3, -15 times tau = 1.5; 0.5, -0.25, 10, -2, 1), so the
    kernels must reproduce the closed form to fp32 accuracy; the reference's bar for this construction
    is 1e-3 (tests/utils/test_linear_cross_entropy.py:392-395)."""
    from verl_amd import linear_cross_entropy

    h, w, y = _two_level_inputs(case, T=5, dtype=dtype, tau=1.5)
    lp, ent = linear_cross_entropy(h.to("cuda:0"), w.to("cuda:0"), y.to("cuda:0"), 1.5, "none")
    want_lp, want_ent = float(case["logprob"]), float(case["entropy"])
    assert lp.cpu().tolist() == pytest.approx([want_lp] * 5, rel=2e-5, abs=2e-6)
    assert ent.cpu().tolist() == pytest.approx([want_ent] * 5, rel=2e-5, abs=2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLD["uniform"], ids=lambda c: f"V{c['V']}")
def test_uniform_logits_kernels(case):
    from verl_amd.utils import torch_functional as F

    V = case["V"]
    z = torch.full((3, V), 0.375, device="cuda:0", dtype=torch.bfloat16)
    ent = F.entropy_from_logits_with_chunking(z)
    lp = F.logprobs_from_logits(z.float(), torch.tensor([0, V // 2, V - 1], device="cuda:0"))
    assert ent.cpu().tolist() == pytest.approx([float(case["entropy"])] * 3, rel=1e-5)
    assert lp.cpu().tolist() == pytest.approx([float(case["logprob"])] * 3, rel=1e-5)


PPO = GOLD["ppo"]
AGG_MODES = ("token-mean", "token-sum", "seq-mean-token-sum", "seq-mean-token-sum-norm", "seq-mean-token-mean")


def _ppo_inputs(device, dtype):
    t = lambda k: torch.tensor(PPO[k], dtype=dtype, device=device)
    return t("log_prob"), t("entropy"), t("old_log_prob"), t("advantages"), t("mask"), t("ref_log_prob")


def test_ppo_oracle_against_the_known_answers():
    """Clipped loss per token (every branch: unclipped, clipped above / below, dual clip, the +-20 clamp), the four KL
    estimators, the five aggregation modes and the masked-mean metrics, evaluated with scalar arithmetic at 40 digits."""
    lp, ent, old, adv, mask, ref = _ppo_inputs("cpu", torch.float64)
    for mode in AGG_MODES:
        pg, met = O.policy_loss_vanilla(old, lp, adv, mask, mode, 0.2, PPO["clip_ratio_low"], PPO["clip_ratio_high"],
                                        PPO["clip_ratio_c"])  # fmt: skip
        assert pg.item() == pytest.approx(float(PPO["pg_loss"][mode]), rel=1e-12)
        assert O.agg_loss(ent, mask, mode).item() == pytest.approx(float(PPO["entropy_loss"][mode]), rel=1e-9)
        for kl in ("kl", "abs", "mse", "low_var_kl"):
            got = O.agg_loss(O.kl_penalty(lp, ref, kl), mask, mode).item()
            assert got == pytest.approx(float(PPO["kl_loss"][kl][mode]), rel=1e-9), (kl, mode)
    assert met["actor/pg_clipfrac"] == pytest.approx(float(PPO["pg_clipfrac"]), rel=1e-9)
    assert met["actor/pg_clipfrac_lower"] == pytest.approx(float(PPO["pg_clipfrac_lower"]), rel=1e-9)
    assert met["actor/ppo_kl"] == pytest.approx(float(PPO["ppo_kl"]), rel=1e-9)
    for kl in ("kl", "abs", "mse", "low_var_kl"):
        want = torch.tensor([[float(v) for v in row] for row in PPO["kl"][kl]], dtype=torch.float64)
        torch.testing.assert_close(O.kl_penalty(lp, ref, kl), want, rtol=1e-12, atol=1e-15)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", AGG_MODES)
@pytest.mark.parametrize("kl", ["kl", "abs", "mse", "low_var_kl"])
def test_ppo_kernels_against_the_known_answers(mode, kl):
    from verl_amd.trainer.ppo.core_algos import agg_loss
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp, ent, old, adv, mask, ref = _ppo_inputs("cuda:0", torch.float32)
    loss, met = fused_ppo_loss(lp, ent, old, adv, mask, clip_ratio_low=PPO["clip_ratio_low"], clip_ratio_high=PPO["clip_ratio_high"],
                               clip_ratio_c=PPO["clip_ratio_c"], entropy_coeff=0.5, loss_agg_mode=mode, ref_log_prob=ref,
                               kl_loss_type=kl, kl_loss_coef=0.25)  # fmt: skip
    pg, el, kll = float(PPO["pg_loss"][mode]), float(PPO["entropy_loss"][mode]), float(PPO["kl_loss"][kl][mode])
    assert met["actor/pg_loss"].item() == pytest.approx(pg, rel=2e-6)
    assert met["actor/entropy_loss"].item() == pytest.approx(el, rel=2e-6)
    assert met["kl_loss"].item() == pytest.approx(kll, rel=2e-6)
    assert loss.item() == pytest.approx(pg - 0.5 * el + 0.25 * kll, rel=2e-6, abs=1e-6)
    assert met["actor/pg_clipfrac"].item() == pytest.approx(float(PPO["pg_clipfrac"]), rel=1e-6)
    assert met["actor/pg_clipfrac_lower"].item() == pytest.approx(float(PPO["pg_clipfrac_lower"]), rel=1e-6)
    assert met["actor/ppo_kl"].item() == pytest.approx(float(PPO["ppo_kl"]), rel=1e-6)
    assert agg_loss(ent, mask, mode).item() == pytest.approx(el, rel=2e-6)
