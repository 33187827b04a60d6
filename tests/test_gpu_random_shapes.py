"""Seeded random shapes through the whole path (C ABI via the autograd wrapper) against the oracle:
ragged token counts, vocabularies that are not multiples of the tile, every hidden size the mainloop
accepts, temperatures, reductions, partly or fully zero upstream gradients, explicit chunk widths.
Tolerances as in tests/test_gpu_lce.py (bf16: the reference's own, fp32: 1e-5 of the largest value)."""

import random

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed):
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float32])
    T = rnd.choice([1, 2, 31, 64, 255, 256, 257, 300, 511, 777, 1024, 1500, 2049])
    H = 128 * rnd.choice([1, 2, 3, 5, 8])
    V = rnd.choice([2, 17, 255, 256, 257, 1000, 4099, 8192, 12345, 20011])
    if seed >= 1000:  # many tokens, ragged against the 256 x 256 tiles of the backward's 16x16x32 loop (the default beyond 1280 tokens)
        T = rnd.choice([4096, 4097, 4500, 5000, 8191, 9001])
        H = 128 * rnd.choice([1, 2, 3])
        V = rnd.choice([255, 257, 1000, 4099, 12345])
    if seed >= 3000:  # 1281 tokens to half a wide hidden size: kept logits feeding the gradient GEMMs of the 16x16x32 loop
        dtype = torch.bfloat16
        H = 128 * rnd.choice([21, 24, 28, 32])
        T = rnd.randint(1281, H // 2)
        V = rnd.choice([257, 1000, 4099, 12345, 20011])
    tau = rnd.choice([0.5, 0.6, 1.0, 1.5, 2.0])
    reduction = rnd.choice(["none", "none", "none", "sum", "mean"])
    mask = rnd.choice(["dense", "dense", "prefix", "random", "zero_lp"])
    vchunk = rnd.choice([0, 0, 256, 1024, 4096])
    return dtype, T, H, V, tau, reduction, mask, vchunk


@pytest.mark.parametrize("seed", range(96))
def test_random_shape(seed):
    _check(seed, None)


@pytest.mark.parametrize("seed", range(96, 128))
def test_random_shape_fp16(seed):
    _check(seed, torch.float16)


@pytest.mark.parametrize("seed", range(1000, 1024))
def test_random_shape_many_tokens(seed):
    _check(seed, torch.float16 if seed % 4 == 3 else None)


@pytest.mark.parametrize("seed", range(3000, 3016))
def test_random_shape_kept_logits_with_many_tokens(seed):
    _check(seed, torch.float16 if seed % 4 == 3 else None)


def _check(seed, force_dtype):
    from verl_amd import linear_cross_entropy
    from verl_amd.utils.kernel import kernels

    dtype, T, H, V, tau, reduction, mask, vchunk = _case(seed)
    dtype = force_dtype or dtype
    g = torch.Generator().manual_seed(1000 + seed)
    h = (torch.rand(T, H, generator=g) - 0.5).to(dtype).to(DEV)
    w = ((torch.rand(V, H, generator=g) - 0.5) * (4.0 / H ** 0.5)).to(dtype).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_ent = (torch.rand(T, generator=g) - 0.5).to(DEV)
    g_lp = (torch.rand(T, generator=g) * 2 - 1).to(DEV) if reduction == "none" else torch.tensor(0.7, device=DEV)
    if mask == "prefix":
        keep = (torch.arange(T) < max(1, T // 3)).to(DEV)
    elif mask == "random":
        keep = (torch.rand(T, generator=g) < 0.4).to(DEV)
    else:
        keep = torch.ones(T, dtype=torch.bool, device=DEV)
    g_ent = g_ent * keep
    if reduction == "none":
        g_lp = g_lp * keep
        if mask == "zero_lp":
            g_lp = torch.zeros_like(g_lp)
    hh = h.clone().requires_grad_(True)
    ww = w.clone().requires_grad_(True)
    try:
        kernels.set_vocab_chunk(vchunk)
        lp, ent = linear_cross_entropy(hh, ww, y, tau, reduction)
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
    finally:
        kernels.set_vocab_chunk(0)
    dh, dw = hh.grad, ww.grad
    assert dh.dtype == dtype and dw.dtype == dtype and dh.shape == h.shape and dw.shape == w.shape
    if dtype == torch.float32:
        rlp, rent = O.lce_forward(h, w, y, tau, reduction, compute_dtype=torch.float64)
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, reduction, compute_dtype=torch.float64)
        for name, got, want in (("lp", lp, rlp), ("ent", ent, rent), ("dh", dh, rdh), ("dw", dw, rdw)):
            err = (got.double() - want).abs().max().item()
            bar = 1e-5 * max(want.abs().max().item(), 1e-3)
            if name == "lp" and reduction == "sum":
                bar = 1e-5 * max(want.abs().max().item(), 1.0) * 4  # a sum of T rounded terms
            assert err <= bar, (name, err, bar, _case(seed))
    else:
        rlp, rent = O.lce_forward(h, w, y, tau, reduction)
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, reduction)
        lp_tol = dict(atol=1e-3 * (T if reduction == "sum" else 1), rtol=2e-4)
        torch.testing.assert_close(lp, rlp, **lp_tol)
        torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
        torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    dead = ~((g_ent != 0) | ((g_lp != 0) if reduction == "none" else torch.ones_like(keep)))
    assert torch.count_nonzero(dh[dead]) == 0
    if T <= H // 2 and dtype != torch.float32:
        # the node kept the forward's logits (no more tokens than half the hidden size); with that switched off
        # the backward recomputes them and must give the same bits
        h2 = h.clone().requires_grad_(True)
        w2 = w.clone().requires_grad_(True)
        try:
            kernels.set_vocab_chunk(vchunk)
            kernels.set_keep_logits_tokens(0)
            lp2, ent2 = linear_cross_entropy(h2, w2, y, tau, reduction)
            torch.autograd.backward([lp2, ent2], [g_lp, g_ent])
        finally:
            kernels.set_keep_logits_tokens(None)
            kernels.set_vocab_chunk(0)
        assert torch.equal(lp, lp2) and torch.equal(ent, ent2)
        assert torch.equal(dh, h2.grad) and torch.equal(dw, w2.grad), _case(seed)
