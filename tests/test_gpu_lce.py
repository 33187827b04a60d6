"""Parity of the HIP path against the oracle, through the Python surface that sits on the C ABI.

Shapes, input distributions and tolerances of the first block are the reference's own
(tests/utils/test_linear_cross_entropy.py:101-163, :219-224, :271-276).  North-star bars are stated
where they are applied: 2e-2 absolute for bf16 inputs, 1e-5 relative for fp32 inputs, on values and
gradients alike.
"""

import math

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def assert_bf16_bar(got, want):
    """North-star bar for bf16 inputs: 2e-2 absolute.  A result that is itself STORED in bf16 cannot
    be closer than half a bf16 ulp of its own magnitude (0.03 for values in [8, 16)), so one bf16 ulp
    (2^-7 relative) of the expected value is allowed on top for the gradients, which are bf16."""
    err = (got.float() - want.float()).abs()
    lim = 2e-2 + 2.0**-7 * want.float().abs()
    assert (err <= lim).all(), f"max err {err.max().item():.3e}, worst excess {(err - lim).max().item():.3e}"


def _uniform_case(T, H, V, dtype, seed, tau=1.5):
    g = torch.Generator().manual_seed(seed)
    h = (torch.rand(T, H, generator=g) - 0.5).to(dtype).to(DEV)
    w = (torch.rand(V, H, generator=g) - 0.5).to(dtype).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_ent = (torch.rand(T, generator=g) - 0.5).to(dtype).to(DEV)
    g_lp = (torch.rand(T, generator=g) * 2 - 1).to(dtype).to(DEV)
    return h, w, y, g_lp, g_ent


def _run(h, w, y, tau, g_lp, g_ent, reduction="none"):
    from verl_amd import linear_cross_entropy

    h = h.clone().requires_grad_(True)
    w = w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(h, w, y, tau, reduction)
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    torch.cuda.synchronize()
    return lp, ent, h.grad, w.grad


REFERENCE_SHAPES = [(1937, 3584, 152064), (2169, 896, 151936), (1530, 2048, 32256), (1388, 4096, 102400),
                    (8192, 4096, 102400)]


@pytest.mark.parametrize("shape", REFERENCE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_reference_shapes_bf16(shape):
    T, H, V = shape
    tau = 1.5
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=T)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau)
    assert lp.dtype == torch.float32 and ent.dtype == torch.float32 and lp.shape == (T,) and ent.shape == (T,)
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
    assert dh.dtype == torch.bfloat16 and dw.dtype == torch.bfloat16 and dh.shape == h.shape and dw.shape == w.shape
    torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    # north-star bar: 2e-2 absolute on values and gradients
    assert (lp - rlp).abs().max() < 2e-2 and (ent - rent).abs().max() < 2e-2
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)


@pytest.mark.parametrize("V", [152064, 149 * 1024])
def test_padded_vocab_known_answer(V):
    """The reference's regression vector (tests/utils/test_linear_cross_entropy.py:352-395): padded
    vocabulary columns must count as -inf, not as logit 0.  Every row: one logit +3, V-1 logits -15."""
    from verl_amd import linear_cross_entropy

    tau, H, T = 1.5, 3584, 512
    w = torch.zeros(V, H, dtype=torch.bfloat16, device=DEV)
    w[:, 0] = -15.0 * tau
    w[0, 0] = 3.0 * tau
    h = torch.zeros(1, T, H, dtype=torch.bfloat16, device=DEV)
    h[:, :, 0] = 1.0
    y = torch.zeros(1, T, dtype=torch.long, device=DEV)
    lp, ent = linear_cross_entropy(h, w, y, tau, "none")
    want_lp, want_ent = O.padded_vocab_known_answer(V)
    assert want_lp == pytest.approx({152064: -0.00231323880878, 152576: -0.00232101851094}[V], rel=1e-9)
    torch.testing.assert_close(lp, torch.full((T,), want_lp, device=DEV), atol=1e-5, rtol=1e-3)
    torch.testing.assert_close(ent, torch.full((T,), want_ent, device=DEV), atol=1e-5, rtol=1e-3)


@pytest.mark.parametrize("shape", [(300, 256, 1000), (1025, 128, 4099), (64, 384, 50257), (2048, 1024, 8192)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("tau", [1.0, 0.6])
def test_fp32_inputs_relative_1e5(shape, tau):
    """fp32 inputs take true-fp32 MFMA; the bar is 1e-5 relative (to the largest magnitude of each
    output) against the oracle evaluated in fp64."""
    T, H, V = shape
    g = torch.Generator().manual_seed(V)
    h = torch.randn(T, H, generator=g).to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.05).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    for got, want in ((lp, rlp), (ent, rent), (dh, rdh), (dw, rdw)):
        assert got.dtype == torch.float32
        err = (got.double() - want).abs().max().item()
        assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())


def test_config1_fp32_forward_and_backward_full_size():
    """The reference's CPU-runnable case (Qwen2.5-0.5B-shaped head, T=1024, H=896, V=151936, fp32, weight
    ~ N(0, 0.02)) at full size: forward to 1e-5 relative against the fp64 oracle, and the backward as well."""
    T, H, V, tau = 1024, 896, 151936, 1.0
    g = torch.Generator().manual_seed(1235)
    h = torch.randn(T, H, generator=g).to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.02).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    for got, want in ((lp, rlp), (ent, rent), (dh, rdh), (dw, rdw)):
        assert got.dtype == torch.float32
        err = (got.double() - want).abs().max().item()
        assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())


@pytest.mark.parametrize("reduction", ["sum", "mean"])
def test_reductions(reduction):
    T, H, V, tau = 700, 256, 3001, 1.3
    h, w, y, _, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=5, tau=tau)
    g_lp = torch.tensor(0.7, device=DEV)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent.float(), reduction)
    rlp, rent = O.lce_forward(h, w, y, tau, reduction)
    assert lp.dim() == 0 and ent.shape == (T,)
    torch.testing.assert_close(lp, rlp, atol=1e-2 if reduction == "sum" else 1e-4, rtol=1e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    rdh, rdw = O.lce_backward(g_lp, g_ent.float(), h, w, y, tau, reduction)
    torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)


def test_profiler_ranges_of_the_reference_bracket_forward_and_backward(monkeypatch):
    """verl/utils/kernel/linear_cross_entropy.py:66,93: the autograd node's forward and backward run inside the ranges
    "LinearCrossEntropy-forward" / "LinearCrossEntropy-backward" (roctx on this platform).  The ranges are pushed and
    popped in pairs, also when the launcher raises, and the results inside them are the oracle's."""
    from verl_amd import linear_cross_entropy

    seen = []
    push, pop = torch.cuda.nvtx.range_push, torch.cuda.nvtx.range_pop
    monkeypatch.setattr(torch.cuda.nvtx, "range_push", lambda name: (seen.append(("push", name)), push(name))[1])
    monkeypatch.setattr(torch.cuda.nvtx, "range_pop", lambda: (seen.append(("pop", None)), pop())[1])
    T, H, V = 300, 128, 1003
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=4)
    h1, w1 = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(h1, w1, y, 0.9, "none")
    assert seen == [("push", "LinearCrossEntropy-forward"), ("pop", None)]
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    assert seen[2:] == [("push", "LinearCrossEntropy-backward"), ("pop", None)]
    rlp, rent = O.lce_forward(h, w, y, 0.9)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, 0.9)
    torch.testing.assert_close(lp, rlp, atol=2e-2, rtol=0)
    torch.testing.assert_close(ent, rent, atol=2e-2, rtol=0)
    torch.testing.assert_close(h1.grad.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(w1.grad.float(), rdw, atol=2e-2, rtol=4e-2)
    # a failing launcher (bad reduction string) still closes its range
    del seen[:]
    with pytest.raises(ValueError):
        linear_cross_entropy(h, w, y, 0.9, "median")
    assert seen == [("push", "LinearCrossEntropy-forward"), ("pop", None)]


def test_api_contract_on_device():
    from verl_amd import linear_cross_entropy
    from verl_amd.utils.kernel import kernels

    T, H, V = 96, 128, 777
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=9)
    # 3-D hidden / 2-D labels: outputs stay flattened, d_hidden is viewed back
    h3 = h.view(2, 48, H).clone().requires_grad_(True)
    w_ = w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(h3, w_, y.view(2, 48), 1.5, "none")
    assert lp.shape == (T,) and ent.shape == (T,)
    # only log-probs used: entropy's gradient arrives as None and must behave as zero
    lp.sum().backward()
    torch.cuda.synchronize()
    assert h3.grad.shape == (2, 48, H) and w_.grad.dtype == torch.bfloat16
    rdh, rdw = O.lce_backward(torch.ones(T, device=DEV), None, h, w, y, 1.5)
    torch.testing.assert_close(h3.grad.float().view(T, H), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(w_.grad.float(), rdw, atol=2e-2, rtol=4e-2)
    # no_grad mode (log-prob passes): same values, no graph
    with torch.no_grad():
        lp2, ent2 = linear_cross_entropy(h, w, y, 1.5, "none")
    assert not lp2.requires_grad
    torch.testing.assert_close(lp2, lp.detach())
    torch.testing.assert_close(ent2, ent.detach())
    # non-contiguous upstream gradients are accepted
    hh = h.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(hh, w, y, 1.5, "none")
    g2 = torch.randn(T, 2, device=DEV)
    torch.autograd.backward([lp, ent], [g2[:, 0], g2[:, 1]])
    rdh, _ = O.lce_backward(g2[:, 0], g2[:, 1], h, w, y, 1.5)
    torch.testing.assert_close(hh.grad.float(), rdh, atol=2e-2, rtol=4e-2)
    # empty micro-batch
    e_lp, e_ent = linear_cross_entropy(h[:0].clone().requires_grad_(True), w_, y[:0], 1.5, "none")
    assert e_lp.shape == (0,) and e_ent.shape == (0,)
    # unsupported pieces fail loudly
    with pytest.raises(NotImplementedError):
        linear_cross_entropy(h, w, y, 1.5, "none", object())

    class OneRank:  # stands for a process group of one rank (Megatron at tensor-parallel size 1)
        def size(self):
            return 1

    g_lp, g_ent = linear_cross_entropy(h, w, y, 1.5, "none", OneRank())
    p_lp, p_ent = linear_cross_entropy(h, w, y, 1.5, "none")
    assert torch.equal(g_lp, p_lp) and torch.equal(g_ent, p_ent)
    with pytest.raises(NotImplementedError):
        linear_cross_entropy(h.double(), w.double(), y, 1.5, "none")
    with pytest.raises(NotImplementedError):
        linear_cross_entropy(h.half(), w, y, 1.5, "none")  # mixed dtypes
    with pytest.raises(AssertionError):
        linear_cross_entropy(h[:, :100].contiguous(), w[:, :100].contiguous(), y, 1.5, "none")  # H % 128
    with pytest.raises(AssertionError):
        linear_cross_entropy(h.t().contiguous().t(), w, y, 1.5, "none")  # non-contiguous hidden
    # out-of-range labels are defined: no label logit, logprob = -logsumexp
    y_bad = y.clone()
    y_bad[0] = -100
    lp_bad, _ = linear_cross_entropy(h, w, y_bad, 1.5, "none")
    z0 = (h[0].float() @ w.float().t()) / 1.5
    assert lp_bad[0].item() == pytest.approx(-torch.logsumexp(z0, -1).item(), abs=1e-3)
    # saved statistics have the reference's meaning
    lp_, ent_, mx, acc, eb = kernels.efficient_entropy_forward(h, w, y, 0, 1.5)
    _, _, rmx, racc, reb = O.lce_forward(h, w, y, 1.5, return_stats=True)
    torch.testing.assert_close(mx, rmx, atol=1e-4, rtol=1e-5)
    torch.testing.assert_close(acc, racc, atol=1e-3, rtol=1e-4)
    torch.testing.assert_close(eb, reb, atol=1e-4, rtol=1e-4)


def _config_case(T, H, V, wstd, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    h = torch.randn(T, H, device=DEV, generator=g).bfloat16()
    w = (torch.randn(V, H, device=DEV, generator=g) * wstd).bfloat16()
    y = torch.randint(0, V, (T,), device=DEV, generator=g)
    g_lp = torch.randn(T, device=DEV, generator=g)
    g_ent = torch.randn(T, device=DEV, generator=g)
    return h, w, y, g_lp, g_ent


def test_config2_full_size_properties_and_sampled_parity():
    """Qwen2.5-7B-shaped head at full size (T=16384, H=3584, V=152064).  The oracle is run on a
    sample of rows for values and d_hidden, and on a slice of vocabulary rows for d_weight;
    size-independent properties cover the rest: sum_v d_weight[v] = 0, log-probs <= 0,
    0 <= entropy <= log V, linearity of the backward in the upstream gradients, determinism."""
    from verl_amd import linear_cross_entropy

    T, H, V, tau = 16384, 3584, 152064, 1.0
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.02, seed=1236)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    assert torch.isfinite(lp).all() and torch.isfinite(ent).all() and torch.isfinite(dh).all() and torch.isfinite(dw).all()
    assert (lp <= 1e-6).all() and (ent >= -1e-4).all() and (ent <= math.log(V) + 1e-4).all()
    rows = torch.arange(0, T, 61, device=DEV)
    rlp, rent = O.lce_forward(h[rows], w, y[rows], tau)
    assert (lp[rows] - rlp).abs().max() < 2e-2 and (ent[rows] - rent).abs().max() < 2e-2
    torch.testing.assert_close(lp[rows], rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent[rows], rent, atol=5e-3, rtol=5e-4)
    rdh, _ = O.lce_backward(g_lp[rows], g_ent[rows], h[rows], w, y[rows], tau)
    assert_bf16_bar(dh[rows], rdh)
    # d_weight needs every token: check it through sum_v dz = 0  =>  sum_v d_weight[v, :] = 0
    col = dw.float().sum(0)
    scale = dw.float().abs().sum(0)
    assert (col.abs() <= 2e-2 * scale + 1e-2).all()
    # and exactly, on a vocabulary slice, against the closed form dz^T h restricted to that slice
    vs = slice(70000, 70256)
    _, _, mx, acc, eb = O.lce_forward(h, w, y, tau, return_stats=True, chunk=2048)
    zs = (h.float() @ w[vs].float().t()) / tau
    p = torch.exp(zs - (mx + acc.log()).unsqueeze(-1))
    dz = -p * g_lp.unsqueeze(-1) - g_ent.unsqueeze(-1) * p * (zs - eb.unsqueeze(-1))
    hit = (y >= vs.start) & (y < vs.stop)
    dz[hit, y[hit] - vs.start] += g_lp[hit]
    want = (dz / tau).t() @ h.float()
    assert_bf16_bar(dw[vs], want)
    # determinism (no float atomics): bit-identical on a second run
    lp2, ent2, dh2, dw2 = _run(h, w, y, tau, g_lp, g_ent)
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2) and torch.equal(dh, dh2) and torch.equal(dw, dw2)


def test_config2_full_size_against_the_whole_oracle():
    """The benchmark's workload itself (Qwen2.5-7B-shaped head, T=16384, H=3584, V=152064, tau=1, dense N(0,1)
    upstream gradients, same seed as bench.py's inputs are drawn from): every log-prob, entropy, d_hidden and
    d_weight entry against the oracle."""
    T, H, V, tau = 16384, 3584, 152064, 1.0
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.02, seed=1236)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau, chunk=2048)
    assert (lp - rlp).abs().max() < 2e-2 and (ent - rent).abs().max() < 2e-2
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    del rlp, rent
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, chunk=2048)
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)
    torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)  # the reference's own tolerance
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)


def test_wide_hidden_and_256k_vocabulary():
    """H = 8192 and V = 262144 (the largest vocabularies in use): 4.3 GB of weights, row offsets beyond
    2^31 bytes inside W, 128 K-slabs per logit tile; a quarter of the tokens without gradient."""
    T, H, V, tau = 2048, 8192, 262144, 0.9
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.01, seed=1241)
    keep = (torch.arange(T, device=DEV) % 4) != 3
    g_lp, g_ent = g_lp * keep, g_ent * keep
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau, chunk=512)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, chunk=512)
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)
    assert (dh[~keep] == 0).all()


def test_config3_masked_rows_temperature_06():
    """Llama-3-8B-shaped head, tau = 0.6, a response mask zeroing a random suffix of each row
    (reduced token count; upstream gradients are zero on masked positions)."""
    H, V, tau = 4096, 128256, 0.6
    rows, L = 4, 512
    T = rows * L
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.02, seed=1237)
    g = torch.Generator().manual_seed(3)
    valid = torch.randint(64, L + 1, (rows,), generator=g)
    mask = (torch.arange(L)[None, :] < valid[:, None]).reshape(-1).to(DEV)
    g_lp, g_ent = g_lp * mask, g_ent * mask
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    assert (lp - rlp).abs().max() < 2e-2 and (ent - rent).abs().max() < 2e-2
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)
    assert (dh[~mask] == 0).all()  # masked tokens receive exactly zero gradient


def test_config4_weight_grad_accumulates_over_many_tokens():
    """Qwen2.5-32B-shaped head (H=5120, V=152064, W ~ N(0, 0.015)); T reduced to 8192 so the oracle
    finishes in seconds.  Exercises d_weight's sum over tokens and several vocabulary chunks."""
    T, H, V, tau = 8192, 5120, 152064, 1.0
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.015, seed=1238)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    assert (lp - rlp).abs().max() < 2e-2 and (ent - rent).abs().max() < 2e-2
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)


def _d_weight_rounding_bound(h, w, y, tau, g_lp, g_ent, rdw, chunk=2048):
    """Bound on |d_weight - exact| that follows from the reference's data format: the gradient of the logits is
    stored in the input dtype before the two GEMMs (verl/utils/kernel/kernels.py:1666-1724: `_d_logits` in
    hidden.dtype), so every dz carries a relative error of up to 2^-9, and d_weight is rounded to bf16 once more:
    |err| <= 2^-9 * (|dz|^T |h|) + 2^-8 * |d_weight|, plus the north-star 2e-2.  Where two tokens with the same
    label pull a weight in opposite directions, |dz|^T |h| is much larger than |d_weight| and a bar relative to
    |d_weight| alone cannot hold with that format."""
    T = h.shape[0]
    _, _, mx, acc, eb = O.lce_forward(h, w, y, tau, return_stats=True, chunk=chunk)
    wf = w.float()
    absdw = torch.zeros_like(rdw)
    for s in range(0, T, chunk):
        e = min(T, s + chunk)
        z = (h[s:e].float() @ wf.t()) / tau
        p = torch.exp(z - (mx[s:e] + acc[s:e].log()).unsqueeze(-1))
        dz = -p * g_lp[s:e].unsqueeze(-1) - g_ent[s:e].unsqueeze(-1) * p * (z - eb[s:e].unsqueeze(-1))
        dz[torch.arange(e - s, device=DEV), y[s:e]] += g_lp[s:e]
        absdw += (dz / tau).abs().t() @ h[s:e].float().abs()
    return 2e-2 + 2.0**-9 * absdw + 2.0**-8 * rdw.abs()


@pytest.mark.parametrize("label_term_outside", [2, 1, 0])
def test_config3_full_size_against_the_whole_oracle(label_term_outside):
    """Llama-3-8B-shaped head at full size: T = 8 x 4096, H=4096, V=128256, tau=0.6, a response mask that zeroes a
    random suffix of each row (valid length U{512..4096}).  Every output is compared with the oracle.  At this
    size some labels occur several times with upstream gradients of opposite sign (d_weight entries of 1.7 that
    are sums of +14 and -12).  By default the one-hot part of d_logits is added in fp32 outside the bf16 tiles and
    the plain bar holds for every entry; with the reference's format (the one-hot part rounded to bf16 inside the
    tile) a few hundred of the 525 M entries exceed it and d_weight is held to that format's rounding bound."""
    from verl_amd import _abi

    H, V, tau = 4096, 128256, 0.6
    rows, L = 8, 4096
    T = rows * L
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.02, seed=1237)
    valid = torch.randint(512, L + 1, (rows,), generator=torch.Generator().manual_seed(3))
    mask = (torch.arange(L)[None, :] < valid[:, None]).reshape(-1).to(DEV)
    g_lp, g_ent = g_lp * mask, g_ent * mask
    lib = _abi.load()
    try:
        assert lib.lce_set_option(4, label_term_outside) == 0
        lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    finally:
        lib.lce_set_option(4, 2)  # the default
    rlp, rent = O.lce_forward(h, w, y, tau, chunk=2048)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, chunk=2048)
    assert (lp - rlp).abs().max() < 2e-2 and (ent - rent).abs().max() < 2e-2
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    assert_bf16_bar(dh, rdh)
    assert (dh[~mask] == 0).all()
    if label_term_outside:
        assert_bf16_bar(dw, rdw)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)  # the reference's own tolerance
    else:
        err = (dw.float() - rdw).abs()
        assert (err <= _d_weight_rounding_bound(h, w, y, tau, g_lp, g_ent, rdw)).all()
        assert int((err > 2e-2 + 2.0**-7 * rdw.abs()).sum()) <= 1000


def test_config4_full_size_against_the_whole_oracle():
    """Qwen2.5-32B-shaped head at full size: T = 32 x 2048, H=5120, V=152064, W ~ N(0, 0.015): d_weight sums over
    65536 tokens, d_hidden over several vocabulary chunks."""
    T, H, V, tau = 65536, 5120, 152064, 1.0
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.015, seed=1238)
    lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rlp, rent = O.lce_forward(h, w, y, tau, chunk=2048)
    assert (lp - rlp).abs().max() < 2e-2 and (ent - rent).abs().max() < 2e-2
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
    del rlp, rent
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, chunk=2048)
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)


@pytest.mark.parametrize("vchunk", [256, 1024, 8192])
def test_vocab_chunking_is_transparent(vchunk):
    from verl_amd.utils.kernel import kernels

    T, H, V, tau = 513, 256, 5000, 1.5
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=11)
    try:
        kernels.set_vocab_chunk(vchunk)
        _, _, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    finally:
        kernels.set_vocab_chunk(0)
    rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
    torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)


@pytest.mark.parametrize("T", [700, 5000])  # the 32x32x16 loop and the 16x16x32 loop
def test_workspace_budget_changes_the_chunking_not_the_result(T):
    """kernels.set_workspace_budget: the backward asks torch for exactly what lce_backward_workspace_bytes reports
    under the budget (peak memory moves with it), runs more, narrower chunks, and returns the same gradients:
    d_weight bit for bit (each row is complete within its chunk), d_hidden to the rounding of one more fp32 sum."""
    from verl_amd import _abi
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    H, V, tau = 512, 40000, 1.0
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=31)
    default_bytes = lib.lce_backward_workspace_bytes(T, H, V, 0, 0)

    def peak_of_one_step():
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        out = _run(h, w, y, tau, g_lp, g_ent)
        return out[2], out[3], torch.cuda.max_memory_allocated() - base

    dh0, dw0, peak_default = peak_of_one_step()
    try:
        kernels.set_workspace_budget(default_bytes // 3)
        small_bytes = lib.lce_backward_workspace_bytes(T, H, V, 0, 0)
        assert small_bytes < default_bytes
        dh1, dw1, peak_small = peak_of_one_step()
    finally:
        kernels.set_workspace_budget(0)
    assert peak_default - peak_small >= 0.8 * (default_bytes - small_bytes)  # the workspace is what shrank
    assert torch.equal(dw0, dw1)
    torch.testing.assert_close(dh0.float(), dh1.float(), atol=1e-3, rtol=2.0**-7)
    rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
    torch.testing.assert_close(dh1.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(dw1.float(), rdw, atol=2e-2, rtol=4e-2)


@pytest.mark.parametrize("T,H,V,vchunk,dtype", [
    (64, 256, 5000, 2048, torch.bfloat16),   # 16 K slices per chunk; the short last chunk leaves half of them empty
    (100, 128, 300, 0, torch.bfloat16),      # single chunk narrower than the slices: empty slices on the first chunk
    (1, 128, 2500, 1024, torch.float32),
    (300, 512, 9000, 0, torch.float32),
])
def test_few_tokens_split_the_d_hidden_reduction(T, H, V, vchunk, dtype):
    """With few tokens the vocabulary reduction of d_hidden is cut into K slices with one fp32 partial
    each (summed in a fixed order at the end); results must not depend on it."""
    from verl_amd.utils.kernel import kernels

    tau = 0.8
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, dtype, seed=19)
    try:
        kernels.set_vocab_chunk(vchunk)
        _, _, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
        _, _, dh2, dw2 = _run(h, w, y, tau, g_lp, g_ent)
    finally:
        kernels.set_vocab_chunk(0)
    if dtype == torch.float32:
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
        for got, want in ((dh, rdh), (dw, rdw)):
            err = (got.double() - want).abs().max().item()
            assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())
    else:
        rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
        torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    assert torch.equal(dh, dh2) and torch.equal(dw, dw2)  # fixed summation order: bit-identical reruns


@pytest.mark.parametrize("pattern", ["prefix", "random", "none", "single", "entropy_only", "first_tile_empty"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_tokens_without_upstream_gradient(pattern, dtype):
    """Prompt and padding positions of a PPO batch arrive with zero upstream gradients.  The backward
    runs on the list of the other tokens only; the result must equal the dense computation (their
    contribution is exactly zero) and d_hidden must be exactly zero on the skipped rows."""
    T, H, V, tau = 1500, 256, 5000, 0.9
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, dtype, seed=23)
    g_lp, g_ent = g_lp.float(), g_ent.float()
    g = torch.Generator().manual_seed(29)
    if pattern == "prefix":       # three packed sequences, each with a masked suffix
        keep = torch.zeros(T, dtype=torch.bool)
        for a, b in ((0, 310), (500, 777), (1000, 1001)):
            keep[a:b] = True
    elif pattern == "random":
        keep = torch.rand(T, generator=g) < 0.3
    elif pattern == "none":
        keep = torch.zeros(T, dtype=torch.bool)
    elif pattern == "single":
        keep = torch.zeros(T, dtype=torch.bool)
        keep[1234] = True
    elif pattern == "entropy_only":  # log-prob gradient zero everywhere, entropy gradient on a few tokens
        keep = torch.rand(T, generator=g) < 0.1
        g_lp = torch.zeros_like(g_lp)
    else:                          # nothing in the first 256-token tile
        keep = torch.ones(T, dtype=torch.bool)
        keep[:300] = False
    keep = keep.to(DEV)
    g_lp, g_ent = g_lp * keep, g_ent * keep
    _, _, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    if dtype == torch.float32:
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
        for got, want in ((dh, rdh), (dw, rdw)):
            err = (got.double() - want).abs().max().item()
            assert err <= 1e-5 * max(want.abs().max().item(), 1e-30), (err, want.abs().max().item())
    else:
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
        torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    dead = ~((g_lp != 0) | (g_ent != 0))
    assert torch.count_nonzero(dh[dead]) == 0
    if pattern == "none":
        assert torch.count_nonzero(dw) == 0


@pytest.mark.parametrize("T,H,V", [(1, 3584, 152064), (64, 3584, 152064), (100, 1024, 128256), (128, 512, 100003), (7, 256, 70)])
def test_few_token_forward_splits_take_contiguous_row_ranges(T, H, V):
    """Up to 128 tokens every vocabulary split of the forward owns one contiguous range of rows whose last tile is
    partial.  Labels are put on the first and last rows of such ranges (multiples of 64 rows and their
    neighbours) and on the last row of the vocabulary, where a wrong range end would drop or double a row."""
    from verl_amd import linear_cross_entropy

    tau = 0.8
    g = torch.Generator().manual_seed(V + T)
    h = torch.randn(T, H, generator=g).bfloat16().to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.03).bfloat16().to(DEV)
    edges = [0, V - 1] + [r + d for r in range(64, V, 64 * max(1, V // 64 // 97)) for d in (-1, 0)]
    y = torch.tensor([edges[i % len(edges)] for i in range(T)], dtype=torch.int64)
    y[T // 2:] = torch.randint(0, V, (T - T // 2,), generator=g)
    y = y.clamp_(0, V - 1).to(DEV)
    with torch.no_grad():
        lp, ent = linear_cross_entropy(h, w, y, tau, "none")
    rlp, rent = O.lce_forward(h, w, y, tau)
    torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
    torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)


@pytest.mark.parametrize("T", [8192, 8193, 9001])
def test_d_hidden_operand_mode_switches_with_token_count(T):
    """Up to 8192 tokens the bf16 d_hidden GEMM reads W as it lies in memory; beyond that it reads a
    transposed copy of each chunk.  Both sides of the switch, ragged and with masked tokens."""
    H, V, tau = 128, 1300, 0.7
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=37)
    g_lp, g_ent = g_lp.float(), g_ent.float()
    keep = (torch.rand(T, generator=torch.Generator().manual_seed(41)) < 0.6).to(DEV)
    g_lp, g_ent = g_lp * keep, g_ent * keep
    _, _, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    assert torch.count_nonzero(dh[~keep]) == 0


@pytest.mark.parametrize("T,V,labels", [(3000, 300, "random"), (700, 5000, "one"), (2500, 1024, "two"), (5000, 70000, "random")])
def test_many_tokens_share_a_label(T, V, labels):
    """The one-hot part of d_weight is summed per label over a label-sorted token list (one workgroup up to 1024
    tokens, several radix passes beyond): labels that repeat tens of times, all tokens on one label, two labels
    with cancelling gradients, and a third of the tokens without gradient; bit-identical on a second run."""
    H, tau = 256, 0.7
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=T + V)
    g_lp, g_ent = g_lp.float() * 4, g_ent.float()
    if labels == "one":
        y = torch.full_like(y, 1234)
    elif labels == "two":
        y = torch.where(torch.arange(T, device=DEV) % 2 == 0, 7, V - 1)
        g_lp = torch.where(torch.arange(T, device=DEV) % 4 < 2, g_lp.abs(), -g_lp.abs())
    keep = (torch.arange(T, device=DEV) % 3) != 1
    g_lp, g_ent = g_lp * keep, g_ent * keep
    _, _, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    assert_bf16_bar(dh, rdh)
    assert_bf16_bar(dw, rdw)
    _, _, dh2, dw2 = _run(h, w, y, tau, g_lp, g_ent)
    assert torch.equal(dh, dh2) and torch.equal(dw, dw2)


def test_every_tile_variant_agrees():
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V, tau = 700, 384, 3001, 1.5
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=13)
    rlp, rent = O.lce_forward(h, w, y, tau)
    rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
    try:
        for v in range(lib.lce_num_variants()):
            assert lib.lce_set_variant(v) == 0
            lp, ent, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
            torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
            torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
            torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
            torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    finally:
        lib.lce_set_variant(-1)


def test_memory_gate_no_T_by_V_tensor():
    """Zero [T, V] logits materialised: peak extra memory of forward and of backward stays below a
    quarter of one bf16 [T, V] tile plus one fp32 [V, H] (the reference's test prints the same peaks,
    tests/utils/test_linear_cross_entropy.py:323-349)."""
    from verl_amd import linear_cross_entropy

    T, H, V, tau = 8192, 2048, 152064, 1.0
    h, w, y, g_lp, g_ent = _config_case(T, H, V, 0.02, seed=17)
    h.requires_grad_(True)
    w.requires_grad_(True)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    lp, ent = linear_cross_entropy(h, w, y, tau, "none")
    torch.cuda.synchronize()
    fwd_peak = torch.cuda.max_memory_allocated() - base
    assert fwd_peak < 64 << 20, fwd_peak  # partial statistics only
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    torch.cuda.synchronize()
    bwd_peak = torch.cuda.max_memory_allocated() - base
    grads = (T * H + V * H) * 2
    assert bwd_peak - grads < 0.25 * T * V * 2 + 4 * V * H, (bwd_peak, grads)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_extreme_logits_closed_forms(dtype):
    """Closed forms at the ends of the numeric range.  (1) Every logit of a token equal (W = 0, or one shared
    weight row so that all logits are -|large|): entropy = log V, logprob = -log V, and d_logits reduces to
    g_lp (1[v=y] - 1/V) / tau, whatever the common value (shift invariance; the reference seeds its running max
    with 0 and loses tokens whose logits are all far below it, verl/utils/kernel/kernels.py:387).
    (2) One logit far above the rest (temperature 0.05): entropy -> 0, logprob of the top label -> 0, of any other
    label = its logit gap; gradients finite and equal to the oracle's."""
    from verl_amd import linear_cross_entropy

    T, H, V = 300, 256, 5003
    g = torch.Generator().manual_seed(4)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    h = torch.ones(T, H, dtype=dtype, device=DEV)
    for fill, tau in ((0.0, 1.0), (-2.0, 0.5)):  # logits 0, and -2 * 256 / 0.5 = -1024 for every vocabulary entry
        w = torch.full((V, H), fill, dtype=dtype, device=DEV)
        hh, ww = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
        lp, ent = linear_cross_entropy(hh, ww, y, tau, "none")
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
        torch.testing.assert_close(ent, torch.full((T,), math.log(V), device=DEV), atol=1e-4, rtol=1e-5)
        torch.testing.assert_close(lp, torch.full((T,), -math.log(V), device=DEV), atol=1e-4, rtol=1e-5)
        dz = -g_lp[:, None].expand(T, V) / V / tau
        want_dw = (dz.double().t() @ h.double())
        want_dw.index_add_(0, y, (g_lp / tau).double()[:, None] * h.double())
        want_dh = fill * (dz.double().sum(1, keepdim=True) + (g_lp / tau).double()[:, None]).expand(T, H)
        tol = dict(atol=2e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=1e-5, rtol=1e-4)
        torch.testing.assert_close(ww.grad.double(), want_dw, **tol)
        # d_hidden is an exact cancellation here (sum_v dz = 0 times a constant weight row).  With 16-bit inputs the
        # V equal softmax terms are rounded to the input format before the GEMM (as the reference's _d_logits is,
        # kernels.py:1666-1724), all in the same direction: allow that format's 2^-8 of the cancelling magnitude.
        # (fp32: 1e-5 relative, of the cancelling magnitude)
        # the entropy term carries (z - b), an exact zero formed from two numbers of size |z| = |fill| H / tau
        rel = 2.0**-8 if dtype == torch.bfloat16 else 1e-5
        slack = rel * abs(fill) * (2 * g_lp.abs() + g_ent.abs() * abs(fill) * H / tau)[:, None] / tau
        assert ((hh.grad.double() - want_dh).abs() <= tol["atol"] + slack).all()
    # (2) a dominant logit: row v of W is e_v-like along one hidden unit per 'class' bucket
    w = torch.zeros(V, H, dtype=dtype, device=DEV)
    w[:, 0] = 0.5
    top = torch.randint(0, V, (T,), generator=g).to(DEV)
    hh = torch.zeros(T, H, dtype=dtype, device=DEV)
    hh[:, 0] = 1.0
    w[torch.arange(256, device=DEV), torch.arange(256, device=DEV) % (H - 1) + 1] = 2.0  # 256 special rows
    sel = torch.arange(T, device=DEV) % 256
    hh[torch.arange(T, device=DEV), sel % (H - 1) + 1] = 3.0  # token t: logit 6.5 on row sel (and its alias row), 0.5 elsewhere
    tau = 0.05  # gaps of 6 / 0.05 = 120 nats
    y2 = torch.where(torch.arange(T, device=DEV) % 2 == 0, sel, top)
    h2, w2 = hh.clone().requires_grad_(True), w.clone().requires_grad_(True)
    lp, ent = linear_cross_entropy(h2, w2, y2, tau, "none")
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    rlp, rent = O.lce_forward(hh, w, y2, tau, compute_dtype=torch.float64)
    rdh, rdw = O.lce_backward(g_lp, g_ent, hh, w, y2, tau, compute_dtype=torch.float64)
    assert torch.isfinite(lp).all() and torch.isfinite(ent).all() and torch.isfinite(h2.grad).all() and torch.isfinite(w2.grad).all()
    torch.testing.assert_close(lp.double(), rlp, atol=1e-3, rtol=1e-5)
    torch.testing.assert_close(ent.double(), rent, atol=1e-4, rtol=1e-4)
    # With 16-bit inputs every softmax term of d_logits, -p (G + g_ent (z - b) / tau), G = g_lp / tau (here up to 60),
    # passes through the 16-bit d_logits format once (up to 2^-8 relative each, as the reference's _d_logits does,
    # kernels.py:1666-1724) while the one-hot part G stays in fp32.  A token that is certain of its label has
    # d_logits[label] = G (1 - p) with p -> 1: that cancellation is then good to the format's rounding of |G p|
    # times |W[label]| (d_hidden) and |h| (the label's row of d_weight).  At the magnitudes of a model
    # (|G| <= 10, |W| <= 0.1) that is below 4e-3.  With fp32 inputs the same cancellation is good to the rounding
    # of p = exp(z - logsumexp) at |z| = 130: a few ulps of |z|, relative.
    z = hh.double() @ w.double().t() / tau
    P = torch.softmax(z, -1)
    bstat = (P * z).sum(-1, keepdim=True)
    soft = P * ((g_lp.abs() / tau).double()[:, None] + (g_ent.abs() / tau).double()[:, None] * (z - bstat).abs())
    rel = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-20 * z.abs().max().item()  # (fp32: ~8 ulps of the log2-domain exponent)
    floor = 2e-2 if dtype == torch.bfloat16 else 1e-5
    # (z - b) of the entropy term is formed in fp32 from two numbers of size |z|: a few ulps of |z| per term
    soft = soft + 2.0**-21 * P * (g_ent.abs() / tau).double()[:, None] * z.abs() * (1.0 / rel)
    bound_dh = floor + rel * rdh.abs() + rel * (soft @ w.double().abs())
    # (d_weight: the softmax terms are rounded to the output format once more before the fp32 one-hot sums are added)
    bound_dw = floor + rel * rdw.abs() + 2 * rel * (soft.t() @ hh.double().abs())
    for name, got, want, bound in (("d_hidden", h2.grad, rdh, bound_dh), ("d_weight", w2.grad, rdw, bound_dw)):
        excess = (got.double() - want).abs() - bound
        i = int(excess.argmax())
        assert excess.max() <= 0, (name, i // H, i % H, got.reshape(-1)[i].item(), want.reshape(-1)[i].item(),
                                   bound.reshape(-1)[i].item())


def test_every_backward_method_runs_and_split_dlogits_m_raises():
    """set_backward_method (verl/utils/kernel/kernels.py:146-180): every BackwardEnum value the reference implements
    gives the oracle's gradients here (they all select the one HIP schedule); _Split_Dlogits_M raises
    NotImplementedError in the backward, as in the reference (:1726-1727)."""
    from verl_amd.utils.kernel import kernels

    T, H, V, tau = 513, 256, 2049, 0.9
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=21)
    rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
    try:
        for method in (kernels.BackwardEnum._Total_Fuse_MN, kernels.BackwardEnum._Total_Separate, kernels.BackwardEnum._Split_Dlogits_N):
            kernels.set_backward_method(method)
            assert kernels._config._backward == method
            _, _, dh, dw = _run(h, w, y, tau, g_lp, g_ent)
            torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
            torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
            assert_bf16_bar(dh, rdh)
            assert_bf16_bar(dw, rdw)
        kernels.set_backward_method(kernels.BackwardEnum._Split_Dlogits_M)
        with pytest.raises(NotImplementedError, match="_Split_Dlogits_M"):
            _run(h, w, y, tau, g_lp, g_ent)
    finally:
        kernels.set_backward_method(kernels.BackwardEnum._Split_Dlogits_N)


@pytest.mark.parametrize("T", [700, 9001])  # the 32x32x16 path and the 16x16x32 path
def test_should_return_fp32_grad_gives_the_fp32_accumulators(T):
    """should_return_fp32_grad (verl/utils/kernel/kernels.py:1562-1567): the gradients leave as fp32 without the final
    rounding to bf16.  They round to exactly what the default call returns (same accumulators, one rounding fewer), and
    they are closer to the oracle than bf16 storage allows: wherever an entry is large enough for its bf16 spacing to
    matter, the fp32 result must beat the bf16 one."""
    from verl_amd.utils.kernel import kernels

    H, V, tau = 256, 3001, 1.1
    h, w, y, g_lp, g_ent = _uniform_case(T, H, V, torch.bfloat16, seed=T)
    lp, ent, mx, acc, eb = kernels.efficient_entropy_forward(h, w, y, 0, tau)
    dh16, dw16 = kernels.efficient_entropy_backward(g_lp.float(), g_ent.float(), h, w, y, mx, acc, eb, 0, False, tau)
    dh32, dw32 = kernels.efficient_entropy_backward(g_lp.float(), g_ent.float(), h, w, y, mx, acc, eb, 0, True, tau)
    assert dh32.dtype == torch.float32 and dw32.dtype == torch.float32 and dh32.shape == (T, H) and dw32.shape == (V, H)
    assert torch.equal(dh32.bfloat16(), dh16)
    # d_weight: equal after rounding on every row that is nobody's label.  On a label's row the 16-bit call rounds
    # twice: the GEMM's sum of the softmax terms first, then that plus the label entries, which are added in fp32
    # (|entry| <= (|g_logprob| + 20 |g_entropy|) / tau per token); the first rounding is half an ulp of the softmax sum
    label_row = torch.zeros(V, dtype=torch.bool, device=DEV)
    label_row[y] = True
    assert torch.equal(dw32.bfloat16()[~label_row], dw16[~label_row])
    entry = torch.zeros(V, H, device=DEV)
    entry.index_add_(0, y, ((g_lp.float().abs() + 20 * g_ent.float().abs()) / tau)[:, None] * h.float().abs())
    slack = 2.0**-7 * dw16.float().abs() + 2.0**-8 * (dw32.abs() + entry)
    assert ((dw32.bfloat16().float() - dw16.float()).abs() <= slack).all()
    rdh, rdw = O.lce_backward(g_lp.float(), g_ent.float(), h, w, y, tau)
    for g32, g16, want in ((dh32, dh16, rdh), (dw32, dw16, rdw)):
        e32, e16 = (g32 - want).abs(), (g16.float() - want).abs()
        assert e32.max() < 2e-2
        assert e32.mean() < e16.mean()
        big = want.abs() > 0.25 * want.abs().max()  # entries whose bf16 spacing is the dominant error of the bf16 result
        assert e32[big].mean() < 0.6 * e16[big].mean(), (e32[big].mean().item(), e16[big].mean().item())
