"""IEEE half-precision inputs (FSDP's param_dtype is configurable, verl/workers/engine/fsdp/transformer_impl.py:391-407):
the same kernels with v_mfma_f32_32x32x16_f16, against the oracle evaluated in fp32 on the fp16-rounded inputs.
Bars: the reference's test tolerances for 16-bit inputs (tests/utils/test_linear_cross_entropy.py:219-224,271-276)
and the 2e-2 absolute bar; gradients are stored in fp16 (2^-10 relative spacing)."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F16 = torch.float16


def _case(T, H, V, seed, wstd=0.02):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, H, generator=g).to(F16).to(DEV)
    w = (torch.randn(V, H, generator=g) * wstd).to(F16).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    return h, w, y, g_lp, g_ent


def _run(h, w, y, tau, g_lp, g_ent):
    from verl_amd import linear_cross_entropy

    h = h.clone().requires_grad_(True)
    w = w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(h, w, y, tau, "none")
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    return lp, ent, h.grad, w.grad


def _check(h, w, y, tau, g_lp, g_ent):
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    assert lp.dtype == torch.float32 and ent.dtype == torch.float32 and dh.dtype == F16 and dw.dtype == F16
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    for got, want in ((lp, rlp), (ent, rent), (dh.float(), rdh), (dw.float(), rdw)):
        assert ((got - want).abs() <= 2e-2 + 2.0**-10 * want.abs()).all()
    return dh, dw


@pytest.mark.parametrize("shape", [(2169, 896, 151936), (1530, 2048, 32256), (777, 256, 5003), (64, 3584, 152064), (9000, 1024, 40000)],
                         ids=lambda s: "x".join(map(str, s)))
def test_fused_head_fp16(shape):
    T, H, V = shape
    h, w, y, g_lp, g_ent = _case(T, H, V, seed=T)
    _check(h, w, y, 1.0 if T != 777 else 0.6, g_lp, g_ent)


def test_fp16_tokens_without_gradient_and_repeated_labels():
    """A response mask (exact zeros required on the skipped rows of d_hidden) and many tokens per label (the one-hot
    term is added in fp32 outside the 16-bit tiles, label rows summed over several tokens)."""
    T, H, V = 4096, 512, 3000
    h, w, y, g_lp, g_ent = _case(T, H, V, seed=3)
    y = y % 17
    mask = (torch.arange(T, device=DEV) % 1024) < 700
    g_lp, g_ent = g_lp * mask, g_ent * mask
    dh, dw = _check(h, w, y, 0.8, g_lp, g_ent)
    assert (dh[~mask] == 0).all()


@pytest.mark.parametrize("shape", [(4, 6, 50), (33, 152064), (2, 7, 4099), (1, 1)])
def test_logits_twins_fp16(shape):
    from verl_amd.utils import torch_functional as F

    g = torch.Generator().manual_seed(shape[-1])
    z = (torch.randn(*shape, generator=g) * 3).to(F16).to(DEV)
    y = torch.randint(0, shape[-1], shape[:-1], generator=g).to(DEV)
    zz = z.clone().requires_grad_(True)
    lp = F.logprobs_from_logits(zz, y)
    ent = F.entropy_from_logits(zz)
    assert lp.dtype == F16 and ent.dtype == F16 and lp.shape == shape[:-1]
    tol = dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(lp.float(), O.logprobs_from_logits(z, y), **tol)
    torch.testing.assert_close(ent.float(), O.entropy_from_logits(z), **tol)
    g_lp = torch.randn(shape[:-1], generator=g).to(F16).to(DEV)
    g_ent = torch.randn(shape[:-1], generator=g).to(F16).to(DEV)
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    want = O.logits_backward(z, y, g_lp.float(), g_ent.float())
    assert zz.grad.dtype == F16 and zz.grad.shape == z.shape
    torch.testing.assert_close(zz.grad.float(), want, **tol)
    got = F.calculate_sum_pi_squared_from_logits(z)
    torch.testing.assert_close(got.double(), O.sum_pi_squared_from_logits(z, torch.float64), **tol)


def test_fused_linear_for_ppo_fp16():
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO

    g = torch.Generator().manual_seed(1)
    B, S, H, V = 2, 300, 96, 1000  # a hidden size that is not a multiple of the K slab
    h = torch.randn(B, S, H, generator=g).to(F16).to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.05).to(F16).to(DEV)
    ids = torch.randint(0, V, (B, S), generator=g).to(DEV)
    lp, ent = FusedLinearForPPO(chunk_size=128)(h, w, ids, temperature=0.7)
    rlp, rent = O.lce_forward(h.reshape(-1, H), w, ids.reshape(-1), 0.7)
    assert lp.shape == (B, S) and ent.dtype == F16
    torch.testing.assert_close(lp.reshape(-1), rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent.reshape(-1).float(), rent, atol=2e-2, rtol=2e-2)
