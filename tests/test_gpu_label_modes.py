"""The three ways the label's entry of d_logits can travel for 16-bit inputs (LCE_OPT_LABEL_TERM_OUTSIDE): 0 = inside
the 16-bit tiles (the reference's data format, verl/utils/kernel/kernels.py:1666-1724), 1 = its one-hot part in fp32
outside the tiles, 2 = the whole entry in fp32 outside the tiles.  Modes 1 and 2 meet the plain bar on ordinary inputs,
mode 0 its format's rounding bound; modes 0 and 1 each have a regime where their rounding shows, mode 2 has neither."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
OPT_LABEL_TERM_OUTSIDE = 4
DEFAULT_MODE = 2


def _run(mode, h, w, y, tau, g_lp, g_ent, vchunk=0):
    from verl_amd import _abi, linear_cross_entropy
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    hh, ww = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    try:
        assert lib.lce_set_option(OPT_LABEL_TERM_OUTSIDE, mode) == 0
        kernels.set_vocab_chunk(vchunk)
        lp, ent = linear_cross_entropy(hh, ww, y, tau, "none")
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
        torch.cuda.synchronize()
    finally:
        kernels.set_vocab_chunk(0)
        lib.lce_set_option(OPT_LABEL_TERM_OUTSIDE, DEFAULT_MODE)
    return hh.grad, ww.grad


def _bar(got, want):
    err = (got.double() - want.double()).abs()
    lim = 2e-2 + 2.0**-7 * want.double().abs()
    i = int((err - lim).argmax())
    assert (err <= lim).all(), (i // got.shape[1], i % got.shape[1], got.reshape(-1)[i].item(), want.reshape(-1)[i].item(), lim.reshape(-1)[i].item())


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,V,vchunk,masked", [(1500, 256, 5003, 0, False), (3000, 512, 300, 0, True), (700, 128, 20011, 4096, True),
                                                (5000, 384, 70000, 0, False), (64, 1024, 32000, 0, False)])
def test_every_mode_against_the_oracle(mode, dtype, T, H, V, vchunk, masked):
    g = torch.Generator().manual_seed(T + mode)
    h = torch.randn(T, H, generator=g).to(dtype).to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.05).to(dtype).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    if masked:  # zero log-prob gradients with live entropy gradients, and tokens without any gradient
        g_lp = g_lp * (torch.arange(T, device=DEV) % 3 != 0)
        dead = torch.arange(T, device=DEV) % 5 == 0
        g_lp, g_ent = g_lp * ~dead, g_ent * ~dead
    dh, dw = _run(mode, h, w, y, 0.8, g_lp, g_ent, vchunk)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, 0.8)
    if mode == 0:
        # the reference's format rounds every one-hot entry G_t to 16 bits inside the tile: where several tokens
        # share a label, their sum in the label's row of d_weight carries 2^-8 of the sum of |G_t h_t|
        G = (g_lp.abs() / 0.8).double()
        slack_dw = torch.zeros(V, H, dtype=torch.float64, device=DEV)
        slack_dw.index_add_(0, y, 2.0**-8 * G[:, None] * h.double().abs())
        slack_dh = 2.0**-8 * G[:, None] * w[y].double().abs()
        assert ((dh.double() - rdh.double()).abs() <= 2e-2 + 2.0**-7 * rdh.double().abs() + slack_dh).all()
        assert ((dw.double() - rdw.double()).abs() <= 2e-2 + 2.0**-7 * rdw.double().abs() + slack_dw).all()
    else:
        _bar(dh, rdh)
        # d_weight: the GEMM's sum of the softmax terms is rounded to 16 bits before the fp32 one-hot sums are added
        # and the row is rounded again; with a vocabulary of 300 those sums are as large as the one-hot ones
        # (-4.77 + 4.75 in one entry here), with a real vocabulary they are small
        G = (g_lp / 0.8).double()
        onehot = torch.zeros(V, H, dtype=torch.float64, device=DEV)
        onehot.index_add_(0, y, G[:, None] * h.double())
        err = (dw.double() - rdw.double()).abs()
        assert (err <= 2e-2 + 2.0**-7 * rdw.double().abs() + 2.0**-8 * (rdw.double() - onehot).abs()).all()
        if V > 1000:
            _bar(dw, rdw)
            torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
            torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    if masked:
        assert (dh[dead] == 0).all()
    dh2, dw2 = _run(mode, h, w, y, 0.8, g_lp, g_ent, vchunk)
    assert torch.equal(dh, dh2) and torch.equal(dw, dw2)  # fixed summation order in every mode


def _certain_label_case():
    """Every token is certain of one vocabulary row (gap of 120 nats at temperature 0.05); even tokens carry that row
    as their label, odd tokens another one.  Weights and gradients are large on purpose (|G| = |g_lp| / tau up to 60)."""
    T, H, V, tau = 300, 256, 5003, 0.05
    g = torch.Generator().manual_seed(4)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    w = torch.zeros(V, H, dtype=torch.bfloat16, device=DEV)
    w[:, 0] = 0.5
    h = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)
    h[:, 0] = 1.0
    r = torch.arange(H - 1, device=DEV)  # 255 special rows, one hidden unit each
    w[r, r + 1] = 2.0
    sel = torch.arange(T, device=DEV) % (H - 1)
    h[torch.arange(T, device=DEV), sel + 1] = 3.0
    other = torch.randint(0, V, (T,), generator=g).to(DEV)
    y = torch.where(torch.arange(T, device=DEV) % 2 == 0, sel, other)
    return h, w, y, tau, g_lp, g_ent


def test_certain_labels_whole_entry_outside_does_not_cancel():
    """d_logits[label] = G (1 - p) with p -> 1.  Mode 1 forms it as G (fp32) minus G p (rounded to 16 bits): an error of
    up to 2^-8 |G W[label]| in d_hidden.  Mode 2 forms it in fp32; what is left is the 16-bit rounding of the OTHER
    entries, which for the even tokens here are all below e^-100."""
    h, w, y, tau, g_lp, g_ent = _certain_label_case()
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    even = torch.arange(h.shape[0], device=DEV) % 2 == 0
    dh1, _ = _run(1, h, w, y, tau, g_lp, g_ent)
    dh2, dw2 = _run(2, h, w, y, tau, g_lp, g_ent)
    err1 = (dh1.double() - rdh).abs()[even].max().item()
    err2 = (dh2.double() - rdh).abs()[even].max().item()
    # fp32 evaluation of p at |z| = 130 leaves a few 1e-3 (ulps of the exponent times |G W| = 120); 16-bit rounding
    # of G p = 60 leaves up to 0.23
    assert err2 <= 5e-3 + 2.0**-8 * rdh.abs()[even].max().item(), err2
    assert err1 <= 2e-2 + 2.0**-8 * 120 and err2 < err1
    # odd tokens: the certain row is not the label, its entry -G p is a large ordinary softmax term in every mode
    z = h.double() @ w.double().t() / tau
    P = torch.softmax(z, -1)
    bstat = (P * z).sum(-1, keepdim=True)
    soft = P * ((g_lp.abs() / tau).double()[:, None] + (g_ent.abs() / tau).double()[:, None] * ((z - bstat).abs() + 2.0**-13 * z.abs()))
    soft[torch.arange(h.shape[0], device=DEV), y] = 0  # the label's entry is outside the tiles
    bound_dh = 5e-3 + 2.0**-8 * rdh.abs() + 2.0**-8 * (soft @ w.double().abs())
    bound_dw = 2e-2 + 2.0**-8 * rdw.abs() + 2.0**-7 * (soft.t() @ h.double().abs())
    assert ((dh2.double() - rdh).abs() <= bound_dh).all()
    assert ((dw2.double() - rdw).abs() <= bound_dw).all()


@pytest.mark.parametrize("mode", [1, 2])
def test_shared_labels_with_cancelling_gradients(mode):
    """Several tokens per label with upstream gradients of opposite sign: a d_weight row is a small difference of
    large one-hot terms.  Inside the 16-bit tiles (mode 0) each term is rounded first; outside they are summed in fp32."""
    T, H, V, tau = 4096, 256, 5000, 0.6
    g = torch.Generator().manual_seed(9)
    h = torch.randn(T, H, generator=g).bfloat16().to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.05).bfloat16().to(DEV)
    y = (torch.randint(0, 8, (T,), generator=g) * 600 + 7).to(DEV)  # eight labels, about 512 tokens each
    g_lp = (torch.randn(T, generator=g) * 4).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    dh, dw = _run(mode, h, w, y, tau, g_lp, g_ent)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
    _bar(dh, rdh)
    # the GEMM's softmax sums of a row are rounded to 16 bits once before the fp32 one-hot sums are added (2^-8 of
    # their size, which is small at a real vocabulary size), then the row is rounded again
    onehot = torch.zeros(V, H, dtype=torch.float64, device=DEV)
    onehot.index_add_(0, y, (g_lp / tau).double()[:, None] * h.double())
    err = (dw.double() - rdw).abs()
    assert (err <= 2e-2 + 2.0**-7 * rdw.abs() + 2.0**-8 * (rdw - onehot).abs()).all()
    # the reference's format on the same input: every one-hot entry rounded on its own
    _, dw0 = _run(0, h, w, y, tau, g_lp, g_ent)
    slack0 = torch.zeros(V, H, dtype=torch.float64, device=DEV)
    slack0.index_add_(0, y, 2.0**-8 * (g_lp.abs() / tau).double()[:, None] * h.double().abs())
    err0 = (dw0.double() - rdw).abs()
    assert (err0 <= 2e-2 + 2.0**-7 * rdw.abs() + slack0).all()
    small = rdw.abs() < 4  # where the output's own 16-bit spacing (2^-6 at most) does not hide the difference
    assert small.any() and err[small].max() < err0[small].max()


def test_option_range():
    from verl_amd import _abi

    lib = _abi.load()
    assert lib.lce_set_option(OPT_LABEL_TERM_OUTSIDE, 3) != 0
    assert lib.lce_set_option(OPT_LABEL_TERM_OUTSIDE, -1) != 0
    assert lib.lce_set_option(OPT_LABEL_TERM_OUTSIDE, DEFAULT_MODE) == 0
