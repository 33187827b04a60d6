"""Vocabulary-parallel building blocks on one GPU: the vocabulary is cut into R shards (uneven, some
not multiples of the tile), every shard runs as its own "rank" one after the other, the partials are
stacked as an all-gather would deliver them, merged, and the shard backwards are summed.  No
collective is involved.  The result must match the unsharded path and the oracle (the reference's TP
test does the same comparison against torch: tests/utils/test_special_linear_cross_entropy_tp.py:128-175)."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _shards(V, R, seed):
    g = torch.Generator().manual_seed(seed)
    if R == 1:
        return [(0, V)]
    cuts = sorted(set(torch.randint(1, V, (R - 1,), generator=g).tolist()))
    edges = [0] + cuts + [V]
    return [(a, b) for a, b in zip(edges[:-1], edges[1:])]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("R", [1, 2, 4, 7])
@pytest.mark.parametrize("reduction", ["none", "mean"])
def test_sharded_equals_unsharded(dtype, R, reduction):
    from verl_amd import linear_cross_entropy
    from verl_amd.utils.kernel import vocab_parallel as VP

    T, H, V, tau = 700, 256, 6007, 0.8
    g = torch.Generator().manual_seed(31 + R)
    h = (torch.rand(T, H, generator=g) - 0.5).to(dtype).to(DEV)
    w = ((torch.rand(V, H, generator=g) - 0.5) * 0.5).to(dtype).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_ent = (torch.rand(T, generator=g) - 0.5).to(DEV)
    g_lp = (torch.rand(T, generator=g) * 2 - 1).to(DEV) if reduction == "none" else torch.tensor(0.6, device=DEV)
    shards = _shards(V, R, seed=R)
    assert len(shards) >= 1 and shards[-1][1] == V
    partials = torch.stack([VP.shard_forward(h, w[a:b].contiguous(), y, a, tau) for a, b in shards])
    lp, ent, mx, acc, eb = VP.merge_shards(partials, reduction)
    # unsharded path
    hh, ww = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    lp0, ent0 = linear_cross_entropy(hh, ww, y, tau, reduction)
    torch.autograd.backward([lp0, ent0], [g_lp, g_ent])
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(lp, lp0.detach(), **(dict(atol=1e-4, rtol=1e-5) if reduction != "none" else tol))
    torch.testing.assert_close(ent, ent0.detach(), **tol)
    # oracle
    rlp, rent = O.lce_forward(h, w, y, tau, reduction, compute_dtype=torch.float64 if dtype == torch.float32 else torch.float32)
    torch.testing.assert_close(lp.double(), rlp.double(), atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent.double(), rent.double(), atol=5e-3, rtol=5e-4)
    # backward: every shard with the merged statistics; d_hidden partials add up, d_weight shards concatenate
    dh = torch.zeros(T, H, device=DEV, dtype=torch.float32)
    dws = []
    for a, b in shards:
        dh_r, dw_r = VP.shard_backward(g_lp, g_ent, h, w[a:b].contiguous(), y, a, mx, acc, eb, reduction, tau)
        dh += dh_r.float()
        dws.append(dw_r)
    dw = torch.cat(dws)
    if dtype == torch.float32:
        for got, want in ((dh, hh.grad), (dw, ww.grad)):
            err = (got.double() - want.double()).abs().max().item()
            assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())
    else:
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, reduction)
        torch.testing.assert_close(dh, rdh, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), ww.grad.float(), atol=2e-2, rtol=4e-2)


def test_label_owned_by_exactly_one_shard():
    """The label logit is reported by the shard that holds the label's row and by no other."""
    from verl_amd.utils.kernel import vocab_parallel as VP

    T, H, V = 64, 128, 1000
    g = torch.Generator().manual_seed(3)
    h = torch.randn(T, H, generator=g).bfloat16().to(DEV)
    w = torch.randn(V, H, generator=g).bfloat16().to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    cut = 437
    p0 = VP.shard_forward(h, w[:cut].contiguous(), y, 0, 1.0)
    p1 = VP.shard_forward(h, w[cut:].contiguous(), y, cut, 1.0)
    z = h.float() @ w.float().t()
    want = z.gather(1, y[:, None]).squeeze(1)
    in0 = y < cut
    torch.testing.assert_close(p0[in0, 3], want[in0], atol=1e-3, rtol=1e-3)
    torch.testing.assert_close(p1[~in0, 3], want[~in0], atol=1e-3, rtol=1e-3)
    assert (p0[~in0, 3] == 0).all() and (p1[in0, 3] == 0).all()
