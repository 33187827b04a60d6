"""Post-head actor step (config 5 shape family, reduced): fused log-prob + entropy feeding the PPO
clipped policy loss with an entropy bonus, forward + backward, against the all-oracle pipeline.
Loss restatement: verl/trainer/ppo/core_algos.py:1140-1206, :1286-1376; verl/workers/utils/losses.py:57-140."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_actor_step_matches_oracle_pipeline():
    from verl_amd import linear_cross_entropy

    H, V, tau = 4096, 128256, 1.0
    nseq, L = 8, 256
    T = nseq * L
    g = torch.Generator(device=DEV).manual_seed(1239)
    h = torch.randn(T, H, device=DEV, generator=g).bfloat16()
    w = (torch.randn(V, H, device=DEV, generator=g) * 0.02).bfloat16()
    y = torch.randint(0, V, (T,), device=DEV, generator=g)
    valid = torch.randint(16, L + 1, (nseq,), device=DEV, generator=g)
    mask = (torch.arange(L, device=DEV)[None, :] < valid[:, None]).float()
    adv = torch.randn(nseq, 1, device=DEV, generator=g).expand(nseq, L).contiguous()
    noise = torch.randn(nseq, L, device=DEV, generator=g) * 0.05

    def pipeline(fused: bool):
        hh = h.clone().requires_grad_(True)
        ww = w.clone().requires_grad_(True)
        if fused:
            lp, ent = linear_cross_entropy(hh, ww, y, tau, "none")
        else:
            z = (hh.float() @ ww.float().t()) / tau
            lp = torch.log_softmax(z, -1).gather(-1, y[:, None]).squeeze(-1)
            ent = torch.logsumexp(z, -1) - (torch.softmax(z, -1) * z).sum(-1)
        lp2, ent2 = lp.view(nseq, L), ent.view(nseq, L)
        old = lp2.detach() + noise
        loss, metrics = O.ppo_actor_loss(lp2, ent2, old, adv, mask, clip_ratio=0.2, entropy_coeff=1e-3)
        loss.backward()
        torch.cuda.synchronize()
        return loss.detach(), metrics, hh.grad.float(), ww.grad.float()

    loss, met, dh, dw = pipeline(True)
    rloss, rmet, rdh, rdw = pipeline(False)
    torch.testing.assert_close(loss, rloss, atol=1e-4, rtol=1e-4)
    for k in ("actor/pg_clipfrac", "actor/ppo_kl", "actor/entropy_loss"):
        assert met[k] == pytest.approx(rmet[k], abs=1e-3, rel=1e-3)
    # token-mean gradients are ~1/N_tokens in size; the absolute bar of 2e-2 is trivially met, so
    # also require agreement relative to the gradient's own scale
    assert (dh - rdh).abs().max() < 2e-2 and (dw - rdw).abs().max() < 2e-2
    assert (dh - rdh).abs().max() <= 2e-2 * rdh.abs().max()
    assert (dw - rdw).abs().max() <= 2e-2 * rdw.abs().max()
