"""``FusedLinearForPPO`` on the GPU, at the cases the reference's own tests use
(tests/utils/test_experimental_torch_functional_on_cpu.py:27-59, :113-124: hidden size 5, vocabulary 11 and 7,
int32 labels, 2-D and 3-D hidden states, temperature 0.7) and at the shape of its sequence-parallel test
(tests/special_distributed/test_fused_kernels_ulysses_sp.py:47-60: hidden 64, vocabulary 256), checked against
the oracle.  Hidden sizes that are not multiples of 128 take the zero-padding route."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("backend", ["torch", "liger", "hip"])
@pytest.mark.parametrize("hidden_shape", [(7, 5), (2, 7, 5)])
def test_tiny_fp32_case_of_the_reference(hidden_shape, backend):
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO

    g = torch.Generator().manual_seed(42)
    tau, V = 0.7, 11
    hidden = torch.randn(hidden_shape, generator=g).to(DEV).requires_grad_(True)
    weight = torch.randn(V, hidden_shape[-1], generator=g).to(DEV).requires_grad_(True)
    labels = torch.randint(V, hidden_shape[:-1], generator=g, dtype=torch.int32).to(DEV)
    g_lp = torch.randn(hidden_shape[:-1], generator=g).to(DEV)
    g_ent = torch.randn(hidden_shape[:-1], generator=g).to(DEV)
    log_probs, entropy = FusedLinearForPPO(impl_backend=backend)(hidden, weight, labels, tau)
    assert log_probs.shape == hidden_shape[:-1] and entropy.shape == hidden_shape[:-1]
    assert entropy.dtype == hidden.dtype
    torch.autograd.backward((log_probs, entropy), (g_lp, g_ent))
    assert hidden.grad.shape == hidden.shape and weight.grad.shape == weight.shape
    rlp, rent = O.lce_forward(hidden.detach(), weight.detach(), labels, tau, compute_dtype=torch.float64)
    rdh, rdw = O.lce_backward(g_lp.double(), g_ent.double(), hidden.detach(), weight.detach(), labels, tau, compute_dtype=torch.float64)
    for got, want in ((log_probs, rlp.reshape(log_probs.shape)), (entropy, rent.reshape(entropy.shape)),
                      (hidden.grad, rdh.reshape(hidden.shape)), (weight.grad, rdw)):
        err = (got.detach().double() - want).abs().max().item()
        assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())


def test_default_temperature_and_forward_only():
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO

    g = torch.Generator().manual_seed(3)
    hidden = torch.randn(2, 3, 5, generator=g).to(DEV)
    weight = torch.randn(7, 5, generator=g).to(DEV)
    labels = torch.randint(7, (2, 3), generator=g).to(DEV)
    log_probs, entropy = FusedLinearForPPO()(hidden, weight, labels)
    rlp, rent = O.lce_forward(hidden, weight, labels, 1.0, compute_dtype=torch.float64)
    torch.testing.assert_close(log_probs.double(), rlp.reshape(2, 3), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(entropy.double(), rent.reshape(2, 3), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_hidden_64_vocabulary_256(dtype):
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO

    g = torch.Generator().manual_seed(11)
    B, S, H, V, tau = 2, 37, 64, 256, 0.9
    hidden = torch.randn(B, S, H, generator=g).to(dtype).to(DEV).requires_grad_(True)
    weight = (torch.randn(V, H, generator=g) * 0.3).to(dtype).to(DEV).requires_grad_(True)
    labels = torch.randint(V, (B, S), generator=g).to(DEV)
    g_lp = torch.randn(B, S, generator=g).to(DEV)
    g_ent = torch.randn(B, S, generator=g).to(DEV)
    log_probs, entropy = FusedLinearForPPO(chunk_size=16)(hidden, weight, labels, tau)
    assert entropy.dtype == dtype and log_probs.dtype == torch.float32
    torch.autograd.backward((log_probs, entropy), (g_lp, g_ent.to(dtype)))
    cd = torch.float64 if dtype == torch.float32 else torch.float32
    rlp, rent = O.lce_forward(hidden.detach(), weight.detach(), labels, tau, compute_dtype=cd)
    rdh, rdw = O.lce_backward(g_lp.to(cd), g_ent.to(dtype).to(cd), hidden.detach(), weight.detach(), labels, tau, compute_dtype=cd)
    if dtype == torch.float32:
        for got, want in ((log_probs, rlp.reshape(B, S)), (entropy, rent.reshape(B, S)), (hidden.grad, rdh.reshape(B, S, H)), (weight.grad, rdw)):
            err = (got.detach().double() - want).abs().max().item()
            assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())
    else:
        torch.testing.assert_close(log_probs, rlp.reshape(B, S), atol=2e-2, rtol=0)
        torch.testing.assert_close(entropy.float(), rent.reshape(B, S), atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(hidden.grad.float(), rdh.reshape(B, S, H), atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(weight.grad.float(), rdw, atol=2e-2, rtol=4e-2)
