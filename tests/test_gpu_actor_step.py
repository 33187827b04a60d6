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


def test_config5_full_size_actor_step_against_the_whole_oracle():
    """The actor micro-step at full size: 64 sequences x 4096 tokens packed to T = 262144, H = 4096, V = 128256,
    response length U{256..4095} per sequence (the rest of each sequence is its prompt), old_log_prob = log_prob +
    N(0, 0.05), one advantage per sequence, clipped loss (0.2, dual clip 3.0, token-mean) minus 1e-3 x token-mean entropy.
    Fused head on the packed tokens -> fused loss on the PACKED outputs (the response slice of no_padding_2_padding,
    verl/workers/utils/padding.py:97-141, applied inside the kernel; gradients come back in packed order) -> fused
    backward, against oracle head (logits materialised 2048 tokens at a time) -> oracle slice -> oracle loss (autograd)
    -> oracle backward; every value and every gradient entry."""
    from verl_amd import linear_cross_entropy
    from verl_amd.workers.utils.losses import fused_ppo_loss_packed

    H, V, tau = 4096, 128256, 1.0
    nseq, L = 64, 4096
    T = nseq * L
    R = L - 1  # max_response_len
    g = torch.Generator(device=DEV).manual_seed(1240)
    h = torch.randn(T, H, device=DEV, generator=g).bfloat16()
    w = (torch.randn(V, H, device=DEV, generator=g) * 0.02).bfloat16()
    y = torch.randint(0, V, (T,), device=DEV, generator=g)
    resp = torch.randint(256, L, (nseq,), device=DEV, generator=g)
    prompt = L - resp
    mask = (torch.arange(R, device=DEV)[None, :] < resp[:, None]).float()
    adv = torch.randn(nseq, 1, device=DEV, generator=g).expand(nseq, R).contiguous()
    noise = torch.randn(nseq, R, device=DEV, generator=g) * 0.05

    rlp, rent = O.lce_forward(h, w, y, tau, chunk=2048)
    old = O.no_padding_2_padding(rlp, prompt.cpu(), resp.cpu(), R) + noise
    hh, ww = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(hh, ww, y, tau, "none")
    assert (lp.detach() - rlp).abs().max() < 2e-2 and (ent.detach() - rent).abs().max() < 2e-2
    torch.testing.assert_close(lp.detach(), rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent.detach(), rent, atol=5e-3, rtol=5e-4)
    loss, met = fused_ppo_loss_packed(lp, ent, prompt, resp, old, adv, mask, clip_ratio=0.2, clip_ratio_c=3.0, entropy_coeff=1e-3)
    loss.backward()
    dh, dw = hh.grad, ww.grad
    del hh, ww, lp, ent
    # oracle slice and loss on the oracle's head outputs; their gradients (packed) feed the oracle's backward
    lp_leaf, ent_leaf = rlp.clone().requires_grad_(True), rent.clone().requires_grad_(True)
    rloss, rmet = O.ppo_actor_loss(O.no_padding_2_padding(lp_leaf, prompt.cpu(), resp.cpu(), R),
                                   O.no_padding_2_padding(ent_leaf, prompt.cpu(), resp.cpu(), R), old, adv, mask, clip_ratio=0.2,
                                   entropy_coeff=1e-3)  # fmt: skip
    rloss.backward()
    torch.testing.assert_close(loss.detach(), rloss.detach(), atol=1e-5, rtol=1e-4)
    for k in ("actor/pg_clipfrac", "actor/ppo_kl", "actor/entropy_loss", "actor/pg_loss"):
        assert met[k].item() == pytest.approx(rmet[k], abs=1e-4, rel=1e-3), k
    rdh, rdw = O.lce_backward(lp_leaf.grad, ent_leaf.grad, h, w, y, tau, chunk=2048)
    # token-mean gradients are ~1/N_tokens in size: require agreement relative to the gradients' own scale
    # (1e-3 of the largest entry plus the bf16 spacing of each entry), far below the absolute bar of 2e-2
    for got, want in ((dh, rdh), (dw, rdw)):
        err = (got.float() - want).abs()
        assert err.max() < 2e-2
        assert (err <= 1e-3 * want.abs().max() + 2.0**-7 * want.abs()).all(), (err.max().item(), want.abs().max().item())
    # tokens that no response position maps to (prompts but for their last token, the last token of each sequence)
    # take no gradient at all
    touched = (lp_leaf.grad != 0) | (ent_leaf.grad != 0)
    assert (dh[~touched] == 0).all() and touched.sum().item() == int(resp.sum().item())
