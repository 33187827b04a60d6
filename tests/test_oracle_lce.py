"""Pins the CPU oracle (oracle/lce_oracle.py, oracle/lce_oracle.c) without touching the GPU.

Each check is chosen so that a plausible mistake (dropped term, wrong sign, transposed operand,
temperature applied on the wrong side) fails at least one of them.
"""

import math

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import lce_oracle as O


def _rand(T, H, V, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, H, generator=g, dtype=dtype)
    w = torch.randn(V, H, generator=g, dtype=dtype) * 0.3
    y = torch.randint(0, V, (T,), generator=g)
    return h, w, y


def _brute(h, w, y, tau):
    """Pure-Python double-precision statement of the definition (tiny inputs only)."""
    T, H = h.shape
    V = w.shape[0]
    lp, ent = [], []
    for t in range(T):
        z = [sum(float(h[t, k]) * float(w[v, k]) for k in range(H)) / tau for v in range(V)]
        m = max(z)
        Z = sum(math.exp(x - m) for x in z)
        p = [math.exp(x - m) / Z for x in z]
        lp.append(math.log(p[int(y[t])]))
        ent.append(-sum(q * math.log(q) for q in p if q > 0))
    return torch.tensor(lp, dtype=torch.float64), torch.tensor(ent, dtype=torch.float64)


# the tiny shapes of the reference's CPU test: tests/utils/test_experimental_torch_functional_on_cpu.py:28-59
@pytest.mark.parametrize("shape", [(7, 5), (2, 7, 5)])
def test_forward_matches_brute_force(shape):
    g = torch.Generator().manual_seed(42)
    V, tau = 11, 0.7
    h = torch.randn(*shape, generator=g, dtype=torch.float64)
    w = torch.randn(V, shape[-1], generator=g, dtype=torch.float64)
    y = torch.randint(0, V, shape[:-1], generator=g, dtype=torch.int32)
    lp, ent = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64)
    blp, bent = _brute(h.reshape(-1, shape[-1]), w, y.reshape(-1), tau)
    assert lp.shape == (math.prod(shape[:-1]),) and ent.shape == lp.shape  # flattened outputs
    torch.testing.assert_close(lp, blp, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(ent, bent, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("V", [152064, 149 * 1024])
def test_padded_vocab_known_answer(V):
    """The reference's regression vector (tests/utils/test_linear_cross_entropy.py:352-395):
    one logit +3, V-1 logits -15, label 0, tau=1.5.  30-digit values quoted from the closed form."""
    ref = {152064: (-0.00231323880878, 0.0439034148162), 152576: (-0.00232101851094, 0.0440509050546)}[V]
    lp_cf, ent_cf = O.padded_vocab_known_answer(V)
    assert lp_cf == pytest.approx(ref[0], rel=1e-10)
    assert ent_cf == pytest.approx(ref[1], rel=1e-10)
    tau, H, T = 1.5, 128, 4
    w = torch.zeros(V, H, dtype=torch.bfloat16)
    w[:, 0] = -15.0 * tau
    w[0, 0] = 3.0 * tau
    h = torch.zeros(T, H, dtype=torch.bfloat16)
    h[:, 0] = 1.0
    y = torch.zeros(T, dtype=torch.long)
    lp, ent = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64)
    torch.testing.assert_close(lp, torch.full((T,), ref[0], dtype=torch.float64), rtol=1e-9, atol=1e-12)
    torch.testing.assert_close(ent, torch.full((T,), ref[1], dtype=torch.float64), rtol=1e-9, atol=1e-12)
    # in fp32 a sequential sum drops the 1.5e-8 terms next to the 1.0 term; the reference's own
    # tolerance for this vector is 1e-3 (tests/utils/test_linear_cross_entropy.py:392-395)
    lp32, ent32 = O.lce_forward(h, w, y, tau)
    torch.testing.assert_close(lp32, torch.full((T,), ref[0]), rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(ent32, torch.full((T,), ref[1]), rtol=1e-3, atol=1e-3)


def test_uniform_logits_closed_form():
    T, H, V = 5, 8, 1000
    h = torch.randn(T, H, dtype=torch.float64)
    w = torch.zeros(V, H, dtype=torch.float64)
    y = torch.arange(T)
    lp, ent = O.lce_forward(h, w, y, 0.5, compute_dtype=torch.float64)
    torch.testing.assert_close(ent, torch.full((T,), math.log(V), dtype=torch.float64))
    torch.testing.assert_close(lp, torch.full((T,), -math.log(V), dtype=torch.float64))


def test_shift_invariance_and_temperature_side():
    h, w, y = _rand(6, 4, 37, seed=3)
    lp, ent = O.lce_forward(h, w, y, 2.0, compute_dtype=torch.float64)
    # adding the same vector c to every weight row shifts all logits of a token by h.c: no change
    c = torch.randn(1, 4, dtype=torch.float64)
    lp2, ent2 = O.lce_forward(h, w + c, y, 2.0, compute_dtype=torch.float64)
    torch.testing.assert_close(lp, lp2)
    torch.testing.assert_close(ent, ent2)
    # temperature divides the logits: tau=2 on h equals tau=1 on h/2
    lp3, ent3 = O.lce_forward(h / 2, w, y, 1.0, compute_dtype=torch.float64)
    torch.testing.assert_close(lp, lp3)
    torch.testing.assert_close(ent, ent3)
    # entropy agrees with scipy's definition
    from scipy.stats import entropy as sp_entropy

    p = torch.softmax(h @ w.t() / 2.0, -1).numpy()
    np.testing.assert_allclose(ent.numpy(), sp_entropy(p, axis=-1), rtol=1e-12)


@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_reductions_and_saved_stats(reduction):
    h, w, y = _rand(9, 4, 23, seed=5)
    lp, ent, m, a, b = O.lce_forward(h, w, y, 1.3, reduction, torch.float64, return_stats=True)
    lp_none, ent_none = O.lce_forward(h, w, y, 1.3, compute_dtype=torch.float64)
    torch.testing.assert_close(ent, ent_none)  # entropy is never reduced
    want = {"none": lp_none, "sum": lp_none.sum(), "mean": lp_none.mean()}[reduction]
    torch.testing.assert_close(lp, want)
    z = h @ w.t() / 1.3
    torch.testing.assert_close(m + a.log(), torch.logsumexp(z, -1))
    torch.testing.assert_close(b, (torch.softmax(z, -1) * z).sum(-1))


def test_bad_reduction():
    h, w, y = _rand(2, 4, 5)
    with pytest.raises(ValueError, match="Invalid reduction"):
        O.lce_forward(h, w, y, 1.0, "max")


@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
@pytest.mark.parametrize("with_entropy", [True, False])
def test_backward_matches_autograd(reduction, with_entropy):
    h, w, y = _rand(6, 5, 13, seed=7)
    tau = 0.7
    h.requires_grad_(True)
    w.requires_grad_(True)
    z = (h @ w.t()) / tau
    lp = torch.log_softmax(z, -1).gather(-1, y[:, None]).squeeze(-1)
    ent = torch.logsumexp(z, -1) - (torch.softmax(z, -1) * z).sum(-1)
    g = torch.Generator().manual_seed(11)
    g_ent = torch.randn(6, generator=g, dtype=torch.float64)
    if reduction == "none":
        g_lp = torch.randn(6, generator=g, dtype=torch.float64)
        loss = (lp * g_lp).sum()
    else:
        g_lp = torch.randn((), generator=g, dtype=torch.float64)
        loss = (lp.sum() if reduction == "sum" else lp.mean()) * g_lp
    if with_entropy:
        loss = loss + (ent * g_ent).sum()
    loss.backward()
    dh, dw = O.lce_backward(g_lp, g_ent if with_entropy else None, h.detach(), w.detach(), y, tau, reduction,
                            torch.float64)
    torch.testing.assert_close(dh, h.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dw, w.grad, rtol=1e-10, atol=1e-12)


def test_unfused_autograd_restatement_equals_the_closed_form():
    """`lce_unfused_autograd` (the reference test's torch path through autograd, which the benchmark times on the GPU as
    context) gives the same four results as the chunked closed form."""
    h, w, y = _rand(7, 6, 19, seed=23)
    tau = 1.3
    g = torch.Generator().manual_seed(5)
    g_lp = torch.randn(7, generator=g, dtype=torch.float64)
    g_ent = torch.randn(7, generator=g, dtype=torch.float64)
    lp, ent, dh, dw = O.lce_unfused_autograd(h, w, y, tau, g_lp, g_ent, torch.float64)
    rlp, rent = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    torch.testing.assert_close(lp, rlp, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(ent, rent, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dh, rdh, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(dw, rdw, rtol=1e-10, atol=1e-12)


def test_backward_finite_differences():
    h, w, y = _rand(3, 4, 9, seed=13)
    tau, eps = 1.5, 1e-6
    g = torch.Generator().manual_seed(2)
    g_lp = torch.randn(3, generator=g, dtype=torch.float64)
    g_ent = torch.randn(3, generator=g, dtype=torch.float64)

    def f(hh, ww):
        lp, ent = O.lce_forward(hh, ww, y, tau, compute_dtype=torch.float64)
        return float((lp * g_lp).sum() + (ent * g_ent).sum())

    dh, dw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    for idx in [(0, 0), (2, 3), (1, 2)]:
        hp, hm = h.clone(), h.clone()
        hp[idx] += eps
        hm[idx] -= eps
        assert (f(hp, w) - f(hm, w)) / (2 * eps) == pytest.approx(float(dh[idx]), rel=1e-6, abs=1e-8)
    for idx in [(0, 0), (8, 3), (int(y[0]), 1)]:
        wp, wm = w.clone(), w.clone()
        wp[idx] += eps
        wm[idx] -= eps
        assert (f(h, wp) - f(h, wm)) / (2 * eps) == pytest.approx(float(dw[idx]), rel=1e-6, abs=1e-8)


def test_backward_invariants():
    """Both gradient terms sum to zero over the vocabulary, so d_hidden is unchanged by adding a
    constant vector to every weight row, and sum_v d_weight[v] = 0."""
    h, w, y = _rand(5, 4, 17, seed=17)
    g_lp = torch.randn(5, dtype=torch.float64)
    g_ent = torch.randn(5, dtype=torch.float64)
    dh, dw = O.lce_backward(g_lp, g_ent, h, w, y, 0.9, compute_dtype=torch.float64)
    torch.testing.assert_close(dw.sum(0), torch.zeros(4, dtype=torch.float64), atol=1e-12, rtol=0)
    dh2, _ = O.lce_backward(g_lp, g_ent, h, w + 3.0, y, 0.9, compute_dtype=torch.float64)
    torch.testing.assert_close(dh, dh2, atol=1e-10, rtol=1e-10)


def test_chunking_is_transparent():
    h, w, y = _rand(37, 8, 29, seed=19, dtype=torch.float32)
    a = O.lce_forward(h, w, y, 1.1, chunk=5)
    b = O.lce_forward(h, w, y, 1.1, chunk=64)
    torch.testing.assert_close(a[0], b[0])
    torch.testing.assert_close(a[1], b[1])
    g = torch.ones(37)
    da = O.lce_backward(g, g, h, w, y, 1.1, chunk=5)
    db = O.lce_backward(g, g, h, w, y, 1.1, chunk=64)
    torch.testing.assert_close(da[0], db[0])
    torch.testing.assert_close(da[1], db[1], rtol=1e-4, atol=1e-5)


def test_c_restatement_agrees_with_torch_restatement():
    h, w, y = _rand(33, 64, 301, seed=23, dtype=torch.float32)
    tau = 1.5
    c = c_oracle.forward(h.numpy(), w.numpy(), y.numpy(), tau)
    lp, ent, m, a, b = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64, return_stats=True)
    np.testing.assert_allclose(c["logprob"], lp.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(c["entropy"], ent.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(c["max"], m.numpy(), rtol=1e-12)
    np.testing.assert_allclose(c["accu"], a.numpy(), rtol=1e-10)
    np.testing.assert_allclose(c["eb"], b.numpy(), rtol=1e-10, atol=1e-12)
    g = torch.Generator().manual_seed(1)
    g_lp = torch.randn(33, generator=g, dtype=torch.float64)
    g_ent = torch.randn(33, generator=g, dtype=torch.float64)
    cdh, cdw = c_oracle.backward(h.numpy(), w.numpy(), y.numpy(), g_lp.numpy(), g_ent.numpy(), tau)
    dh, dw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    np.testing.assert_allclose(cdh, dh.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(cdw, dw.numpy(), rtol=1e-9, atol=1e-12)


def test_logits_functions():
    g = torch.Generator().manual_seed(29)
    z = torch.randn(4, 6, 50, generator=g, dtype=torch.float64) * 3
    y = torch.randint(0, 50, (4, 6), generator=g)
    lp = O.logprobs_from_logits(z, y, torch.float64)
    ent = O.entropy_from_logits(z, torch.float64)
    p = torch.softmax(z, -1)
    torch.testing.assert_close(lp, torch.log(p.gather(-1, y[..., None]).squeeze(-1)))
    torch.testing.assert_close(ent, -(p * p.log()).sum(-1))
    # +-1000 logits stay finite (cf. tests/utils/test_torch_functional.py:126-150)
    big = torch.tensor([[1000.0, -1000.0, 0.0]], dtype=torch.float32)
    assert torch.isfinite(O.entropy_from_logits(big)).all()
    assert O.logprobs_from_logits(big, torch.tensor([0])).item() == pytest.approx(0.0, abs=1e-6)
    # gradient restatement vs autograd
    zz = z.clone().requires_grad_(True)
    g_lp = torch.randn(4, 6, generator=g, dtype=torch.float64)
    g_ent = torch.randn(4, 6, generator=g, dtype=torch.float64)
    loss = (O.logprobs_from_logits(zz, y, torch.float64) * g_lp).sum() + (
        O.entropy_from_logits(zz, torch.float64) * g_ent
    ).sum()
    loss.backward()
    torch.testing.assert_close(O.logits_backward(z, y, g_lp, g_ent, torch.float64), zz.grad)
    torch.testing.assert_close(O.logits_backward(z, y, g_lp, None, torch.float64).sum(-1), torch.zeros(4, 6,
                               dtype=torch.float64), atol=1e-12, rtol=0)


def test_sum_pi_squared_closed_forms_and_brute_force():
    """Pins ``sum_pi_squared_from_logits`` (verl/utils/torch_functional.py:687-703) without retyping its
    formula: uniform logits give 1/V, one logit raised by log(1/r) over V-1 equal ones gives
    (1 + (V-1) r^2) / (1 + (V-1) r)^2, a dominant logit gives 1, and small random rows are summed in pure Python."""
    import math

    for V in (1, 2, 7, 1000):
        z = torch.full((3, V), 4.25, dtype=torch.float64)
        torch.testing.assert_close(O.sum_pi_squared_from_logits(z, torch.float64), torch.full((3,), 1.0 / V, dtype=torch.float64))
    V, r = 50, 0.125
    z = torch.full((1, V), -2.0, dtype=torch.float64)
    z[0, 17] += math.log(1 / r)
    want = (1 + (V - 1) * r * r) / (1 + (V - 1) * r) ** 2
    assert O.sum_pi_squared_from_logits(z, torch.float64).item() == pytest.approx(want, rel=1e-12)
    big = torch.tensor([[1000.0, -1000.0, 0.0]])
    assert O.sum_pi_squared_from_logits(big).item() == pytest.approx(1.0, abs=1e-6)
    g = torch.Generator().manual_seed(31)
    z = torch.randn(5, 9, generator=g, dtype=torch.float64) * 2
    for row, got in zip(z.tolist(), O.sum_pi_squared_from_logits(z, torch.float64).tolist()):
        mx = max(row)
        e = [math.exp(v - mx) for v in row]
        s = sum(e)
        assert got == pytest.approx(sum((v / s) ** 2 for v in e), rel=1e-12)
    # shift invariance, and the shape contract (last dimension reduced)
    torch.testing.assert_close(O.sum_pi_squared_from_logits(z + 3.0, torch.float64), O.sum_pi_squared_from_logits(z, torch.float64))
    assert O.sum_pi_squared_from_logits(torch.zeros(2, 3, 4)).shape == (2, 3)
