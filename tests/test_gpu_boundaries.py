"""Deterministic cases ON the discontinuities and at the rounding limits that a random sweep only hits by chance.

A sweep of 600 random PPO batches against the fp64 oracle left four single-element gradient mismatches; all four sit at a
probability ratio within 2e-8 of a clip boundary (log-ratio = the fp32 neighbour of log 1.2 or log 0.8): in fp64 the
ratio is just inside the clip range (gradient -A * ratio), in fp32 just outside (gradient 0).  At a discontinuity both
one-sided values are correct answers (and exactly on a tie their mean, which is what torch's autograd returns there);
what must never happen is anything else.  The same sweep left seven fp32
logits-twin cases 2e-5..6e-5 off at logits of scale 30: log-prob = z_label - logsumexp is a difference of two numbers of
size max|z|, so its absolute error is a few ulps OF max|z| however small the result is (torch's own fp32 log_softmax has
the same limit)."""

import math

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _neighbours(x: float, n: int = 2):
    """the fp32 numbers around x: x rounded, and n steps to either side"""
    t = torch.tensor(x, dtype=torch.float32)
    out = [t.item()]
    up, dn = t.clone(), t.clone()
    for _ in range(n):
        up = torch.nextafter(up, torch.tensor(float("inf")))
        dn = torch.nextafter(dn, torch.tensor(float("-inf")))
        out += [up.item(), dn.item()]
    return out


@pytest.mark.parametrize("mode", ["token-sum", "token-mean"])
def test_ppo_gradient_on_the_clip_boundaries_is_one_of_the_two_sides(mode):
    from verl_amd.workers.utils.losses import fused_ppo_loss

    # log-ratios on and next to every kink of the vanilla loss: clip at 1 - 0.2 and 1 + 0.2, dual clip at ratio = 3,
    # the +-20 clamp of the log-ratio, and ratio = 1
    ds = []
    for x in (math.log(0.8), math.log(1.2), math.log(3.0), 20.0, -20.0, 0.0):
        ds += _neighbours(x)
    d = torch.tensor(ds, dtype=torch.float32)
    n = d.numel()
    advs = torch.tensor([1.0, -1.0, 0.37, -2.5, 0.0])
    lp = (-torch.rand(advs.numel(), n, generator=torch.Generator().manual_seed(0))).to(DEV)
    old = (lp.cpu() - d[None, :]).to(DEV)  # log-ratio = lp - old (exactly d wherever the subtraction is exact; near it otherwise)
    adv = advs[:, None].expand(-1, n).contiguous().to(DEV)
    mask = torch.ones_like(lp)
    lp1 = lp.clone().requires_grad_(True)
    loss, _ = fused_ppo_loss(lp1, None, old, adv, mask, clip_ratio=0.2, clip_ratio_c=3.0, loss_agg_mode=mode)
    loss.backward()
    got = lp1.grad.double()
    # both one-sided gradients from the fp64 oracle, with the log-ratio nudged off the kink by 1e-6 either way
    sides = []
    for eps in (-1e-6, 1e-6):
        lp2 = (lp.double() + eps).requires_grad_(True)
        rl, _ = O.ppo_actor_loss(lp2, None, old.double(), adv.double(), mask.double(), clip_ratio=0.2, loss_agg_mode=mode)
        rl.backward()
        sides.append(lp2.grad)
    scale = max(s.abs().max().item() for s in sides)
    near = lambda a, b: (a - b).abs() <= 3e-5 * b.abs() + 3e-6 * scale  # noqa: E731
    # (exactly ON a tie torch.maximum / torch.min split the gradient evenly: the mean of the two sides)
    ok = near(got, sides[0]) | near(got, sides[1]) | near(got, 0.5 * (sides[0] + sides[1]))
    assert ok.all(), (got[~ok], sides[0][~ok], sides[1][~ok])
    assert torch.isfinite(loss)


def test_ppo_kl_abs_at_equal_log_probs_and_zero_advantage():
    """|log_prob - ref_log_prob| has its kink at equality: the reference's autograd gives sign(0) = 0 there, and so does
    the kernel; a zero advantage makes both clip branches tie (l1 = l2 = 0) and the gradient exactly zero."""
    from verl_amd.workers.utils.losses import fused_ppo_loss

    lp = torch.tensor([[-1.0, -0.5, -2.0, -0.25]], device=DEV)
    ref = torch.tensor([[-1.0, -0.5000001, -2.0, -0.2499999]], device=DEV)
    old = lp.clone()
    adv = torch.zeros_like(lp)
    mask = torch.ones_like(lp)
    lp1 = lp.clone().requires_grad_(True)
    loss, met = fused_ppo_loss(lp1, None, old, adv, mask, ref_log_prob=ref, kl_loss_type="abs", kl_loss_coef=1.0, loss_agg_mode="token-sum")
    loss.backward()
    lp2 = lp.double().requires_grad_(True)
    rl, _ = O.ppo_actor_loss(lp2, None, old.double(), adv.double(), mask.double(), ref_log_prob=ref.double(), kl_loss_type="abs",
                             kl_loss_coef=1.0, loss_agg_mode="token-sum")
    rl.backward()
    assert lp1.grad.tolist() == [[0.0, 1.0, 0.0, -1.0]] and lp2.grad.tolist() == [[0.0, 1.0, 0.0, -1.0]]
    torch.testing.assert_close(loss.double(), rl.detach(), atol=1e-9, rtol=1e-6)


@pytest.mark.parametrize("V", [65, 4099, 152064])
def test_fp32_logits_twins_error_scales_with_the_largest_logit(V):
    """fp32 twins at logits of scale 30 (max |z| around 130): |error| <= 2e-5 + 4 ulp(max |z|) against the fp64 oracle,
    for log-probs and entropies of any size; at scale 0.1 the plain 2e-5 bar holds."""
    from verl_amd.utils import torch_functional as F

    g = torch.Generator().manual_seed(V)
    for scale in (0.1, 30.0):
        z = (torch.randn(64, V, generator=g) * scale).to(DEV)
        y = torch.randint(0, V, (64,), generator=g).to(DEV)
        lp, ent = F.logprobs_from_logits(z, y), F.entropy_from_logits(z)
        want_lp = O.logprobs_from_logits(z, y, compute_dtype=torch.float64)
        want_ent = O.entropy_from_logits(z, compute_dtype=torch.float64)
        bound = 2e-5 + 4 * 2.0**-23 * z.abs().amax(dim=-1).double()
        assert ((lp.double() - want_lp).abs() <= bound).all(), ((lp.double() - want_lp).abs().max().item(), bound.min().item())
        assert ((ent.double() - want_ent).abs() <= bound).all(), ((ent.double() - want_ent).abs().max().item(), bound.min().item())
        if scale == 0.1:
            assert (lp.double() - want_lp).abs().max() <= 2e-5 and (ent.double() - want_ent).abs().max() <= 2e-5
