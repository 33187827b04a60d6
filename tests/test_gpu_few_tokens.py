"""Backward with at most 128 tokens and 16-bit inputs: both gradient GEMMs run as streaming kernels (one launch,
d_weight rows written once in 64-byte runs, d_hidden from fp32 K-slice partials with W read in place) instead of
the 256 x 256 tile kernels.  Same bar as every other backward (verl/utils/kernel/kernels.py:1380-1515,1666-1724 is
the reference's schedule for these two products): 2e-2 absolute for bf16 against the oracle, bit-identical reruns,
and agreement with the tile kernels that LCE_OPT_FEW_TOKEN_GEMMS = 0 selects."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
OPT_FEW_TOKEN_GEMMS = 9


def _case(T, H, V, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, H, generator=g).to(dtype).to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.05).to(dtype).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = torch.randn(T, generator=g).to(DEV)
    g_ent = torch.randn(T, generator=g).to(DEV)
    return h, w, y, g_lp, g_ent


def _run(h, w, y, tau, g_lp, g_ent, few=1, vchunk=0, fp32_grad=False):
    from verl_amd import _abi, linear_cross_entropy
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    hh, ww = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    try:
        assert lib.lce_set_option(OPT_FEW_TOKEN_GEMMS, few) == 0
        kernels.set_vocab_chunk(vchunk)
        if fp32_grad:
            lp, ent, mx, acc, eb = kernels.efficient_entropy_forward(h, w, y, 0, tau)
            dh, dw = kernels.efficient_entropy_backward(g_lp, g_ent, h, w, y, mx, acc, eb, 0, True, tau)
        else:
            lp, ent = linear_cross_entropy(hh, ww, y, tau, "none")
            torch.autograd.backward([lp, ent], [g_lp, g_ent])
            dh, dw = hh.grad, ww.grad
        torch.cuda.synchronize()
    finally:
        kernels.set_vocab_chunk(0)
        lib.lce_set_option(OPT_FEW_TOKEN_GEMMS, 1)
    return dh, dw


def _bar(got, want):
    err = (got.double() - want.double()).abs()
    lim = 2e-2 + 2.0**-7 * want.double().abs()
    assert (err <= lim).all(), (err.max().item(), (err - lim).max().item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,V,vchunk", [
    (1, 256, 5003, 0),        # one token: 63 zero rows pad the reduction of d_weight
    (17, 3584, 20011, 0),     # vocabulary that is no multiple of the 64-column blocks, hidden of 14 column tiles
    (64, 384, 50257, 0),      # hidden of one and a half column tiles
    (64, 128, 32000, 4096),   # eight chunks: the d_hidden partials of later chunks are added to the first chunk's
    (65, 1024, 32000, 0),     # just past 64 tokens: the 128-position kernels
    (100, 2048, 128256, 0),
    (128, 512, 100003, 8192),
    (128, 128, 300, 0),       # a hidden narrower than a tile, a vocabulary narrower than the K slices
])
def test_against_the_oracle_and_the_tile_kernels(T, H, V, vchunk, dtype):
    tau = 0.8
    h, w, y, g_lp, g_ent = _case(T, H, V, dtype, seed=T + H)
    dh, dw = _run(h, w, y, tau, g_lp, g_ent, few=1, vchunk=vchunk)
    dh_again, dw_again = _run(h, w, y, tau, g_lp, g_ent, few=1, vchunk=vchunk)
    dh_tiles, dw_tiles = _run(h, w, y, tau, g_lp, g_ent, few=0, vchunk=vchunk)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    _bar(dh, rdh)
    _bar(dw, rdw)
    assert torch.equal(dh, dh_again) and torch.equal(dw, dw_again)  # fixed summation order
    # the two code paths sum d_weight over the same tokens in fp32 and round once: equal up to one 16-bit ulp
    ulp = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    assert ((dw.float() - dw_tiles.float()).abs() <= 1e-6 + ulp * dw_tiles.float().abs()).all()
    assert ((dh.float() - dh_tiles.float()).abs() <= 2e-3 + 2 * ulp * dh_tiles.float().abs()).all()


@pytest.mark.parametrize("T", [40, 120])
@pytest.mark.parametrize("pattern", ["none", "single", "sparse", "tail"])
def test_tokens_without_upstream_gradient(T, pattern):
    """The token list is built on the device; the streaming kernels read its length there: k-steps of d_weight
    beyond it are skipped (those rows of the compact hidden copy are not initialised), d_hidden rows of skipped
    tokens are exactly zero."""
    H, V, tau = 512, 30011, 0.9
    h, w, y, g_lp, g_ent = _case(T, H, V, torch.bfloat16, seed=7 + T)
    keep = torch.zeros(T, dtype=torch.bool, device=DEV)
    if pattern == "single":
        keep[T // 2] = True
    elif pattern == "sparse":
        keep[::7] = True
    elif pattern == "tail":
        keep[T - 33:] = True
    g_lp, g_ent = g_lp * keep, g_ent * keep
    dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    _bar(dh, rdh)
    _bar(dw, rdw)
    assert torch.count_nonzero(dh[~keep]) == 0
    if pattern == "none":
        assert torch.count_nonzero(dw) == 0 and torch.count_nonzero(dh) == 0


@pytest.mark.parametrize("T", [64, 128])
def test_fp32_gradients(T):
    """should_return_fp32_grad: the streaming kernels write the fp32 accumulators of d_weight; they round to what the
    16-bit call returns and are closer to the oracle on average."""
    H, V, tau = 1024, 50257, 1.0
    h, w, y, g_lp, g_ent = _case(T, H, V, torch.bfloat16, seed=3)
    dh32, dw32 = _run(h, w, y, tau, g_lp, g_ent, fp32_grad=True)
    dh16, dw16 = _run(h, w, y, tau, g_lp, g_ent)
    assert dh32.dtype == torch.float32 and dw32.dtype == torch.float32
    assert torch.equal(dh32.bfloat16(), dh16)
    # d_weight: the same accumulators, so equal after rounding, except on the rows of the labels, where the 16-bit call
    # rounds twice (the softmax terms, then their sum with the one-hot terms that are added in fp32): one ulp of the
    # result there, or half an ulp of the softmax terms where the two parts cancel (entries of 1e-4 off by 1e-6; bound 2e-4)
    label_row = torch.zeros(V, dtype=torch.bool, device=DEV)
    label_row[y] = True
    assert torch.equal(dw32.bfloat16()[~label_row], dw16[~label_row])
    assert ((dw32.bfloat16().float() - dw16.float()).abs() <= 2e-4 + 2.0**-7 * dw16.float().abs())[label_row].all()
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    assert (dw32 - rdw).abs().mean() < (dw16.float() - rdw).abs().mean()


def test_full_vocabulary_config2_head():
    """qwen2.5-7b head (H=3584, V=152064) at 64 tokens, the shape the few-token bench line is quoted on: both gradients
    whole against the oracle."""
    T, H, V, tau = 64, 3584, 152064, 1.0
    h, w, y, g_lp, g_ent = _case(T, H, V, torch.bfloat16, seed=11)
    dh, dw = _run(h, w, y, tau, g_lp, g_ent)
    rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
    _bar(dh, rdh)
    _bar(dw, rdw)


@pytest.mark.parametrize("label_mode", [2, 1, 0])
@pytest.mark.parametrize("T,H,V,vchunk,reduction", [
    (1, 256, 5003, 0, 0),
    (17, 3584, 20011, 0, 0),
    (64, 128, 32000, 4096, 1),   # eight chunks: each takes its rows of the kept logits
    (65, 1024, 32000, 0, 2),
    (128, 512, 100003, 8192, 0),
    (128, 256, 300, 0, 0),
    (129, 256 + 128, 20011, 0, 0),  # beyond 128 tokens: the 256-token tiles write the logits, the tile GEMMs read d_logits
    (300, 640, 50257, 8192, 2),  # two token tiles, seven chunks
    (512, 1024, 30000, 0, 1),
    (513, 1152, 9001, 0, 0),     # beyond 512 tokens the 16x16x32 forward tiles write the logits
    (1000, 2048, 20011, 4096, 2),
    (1280, 2560, 5003, 0, 1),
    (1281, 2688, 5003, 0, 0),    # beyond 1280 tokens the backward's tiles are those of the 16x16x32 loop (groups of 128 vocabulary rows)
    (1500, 3584, 12007, 4096, 2),
    (1792, 3584, 9001, 0, 1),
    (2048, 4096, 3001, 2048, 0),
])
def test_backward_from_kept_logits_is_bit_identical(T, H, V, vchunk, reduction, label_mode):
    """With few tokens (at most half the hidden size) the forward can keep its fp32 logits and the backward then computes d_logits from them
    instead of from a pass over W: same outputs from the forward, same bits in both gradients (16-bit and fp32), with
    tokens without gradient, labels outside the vocabulary, every reduction and every format of the label's entry."""
    from verl_amd import _abi
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    tau = 0.7
    h, w, y, g_lp, g_ent = _case(T, H, V, torch.bfloat16, seed=T + V)
    y[::5] = -100                       # ignored labels
    g_lp[1::3] = 0.0
    g_ent[1::3] = 0.0                   # tokens without upstream gradient
    g = g_lp if reduction == 0 else g_lp[:1].reshape(())
    try:
        assert lib.lce_set_option(4, label_mode) == 0
        kernels.set_vocab_chunk(vchunk)
        plain = kernels.efficient_entropy_forward(h, w, y, reduction, tau)
        *kept, cache = kernels.forward_keeping_logits(h, w, y, reduction, tau)
        assert cache is not None and cache.numel() == T * ((V + 63) // 64 * 64) * 4
        for a, b in zip(plain, kept):
            assert torch.equal(a, b)
        mx, acc, eb = plain[2:]
        for fp32 in (True, False):
            dh0, dw0 = kernels.efficient_entropy_backward(g, g_ent, h, w, y, mx, acc, eb, reduction, fp32, tau)
            dh1, dw1 = kernels.efficient_entropy_backward(g, g_ent, h, w, y, mx, acc, eb, reduction, fp32, tau, logits_cache=cache)
            assert torch.equal(dh0, dh1) and torch.equal(dw0, dw1)
        only_dh, none = kernels.efficient_entropy_backward(g, g_ent, h, w, y, mx, acc, eb, reduction, False, tau,
                                                           need_d_weight=False, logits_cache=cache)
        assert none is None and torch.equal(only_dh, dh1)
        torch.cuda.synchronize()
    finally:
        kernels.set_vocab_chunk(0)
        lib.lce_set_option(4, 2)


@pytest.mark.parametrize("T,H,V", [(100, 512, 20011), (700, 2048, 9001), (1500, 3072, 12007)])
def test_backward_from_kept_logits_is_bit_identical_in_fp16(T, H, V):
    """fp16 has exact ties where bf16 has few (a product of two short mantissas that lands on the middle of two fp16
    values): both ways to d_logits round once, from the same fp32 value, in every kernel that writes them."""
    from verl_amd.utils.kernel import kernels

    h, w, y, g_lp, g_ent = _case(T, H, V, torch.float16, seed=3 * T + V)
    *out, cache = kernels.forward_keeping_logits(h, w, y, 0, 0.5)
    assert cache is not None
    mx, acc, eb = out[2:]
    for fp32 in (True, False):
        dh0, dw0 = kernels.efficient_entropy_backward(g_lp, g_ent, h, w, y, mx, acc, eb, 0, fp32, 0.5)
        dh1, dw1 = kernels.efficient_entropy_backward(g_lp, g_ent, h, w, y, mx, acc, eb, 0, fp32, 0.5, logits_cache=cache)
        assert torch.equal(dh0, dh1) and torch.equal(dw0, dw1)
    torch.cuda.synchronize()


def test_no_logits_are_kept_beyond_half_the_hidden_size_or_for_fp32():
    from verl_amd import _abi
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    assert lib.lce_logits_cache_bytes(128, 512, 1000, _abi.DTYPE_BF16) == 128 * 1024 * 4
    assert lib.lce_logits_cache_bytes(256, 512, 1000, _abi.DTYPE_BF16) == 256 * 1024 * 4   # as large as the weight: the most
    assert lib.lce_logits_cache_bytes(257, 512, 1000, _abi.DTYPE_BF16) == 0
    assert lib.lce_logits_cache_max_tokens(512, _abi.DTYPE_BF16) == 256
    assert lib.lce_logits_cache_max_tokens(3584, _abi.DTYPE_F16) == 1792
    assert lib.lce_logits_cache_bytes(2048, 4096, 1000, _abi.DTYPE_BF16) == 2048 * 1024 * 4
    assert lib.lce_logits_cache_bytes(2049, 4096, 1000, _abi.DTYPE_BF16) == 0
    assert lib.lce_logits_cache_bytes(64, 512, 1000, _abi.DTYPE_F32) == 0 and lib.lce_logits_cache_max_tokens(512, _abi.DTYPE_F32) == 0
    h, w, y, g_lp, g_ent = _case(513, 256, 3000, torch.bfloat16, seed=1)
    assert kernels.forward_keeping_logits(h, w, y, 0, 1.0)[5] is None
    # a buffer where none is used, and one that is too small, are refused before anything is launched
    buf = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    f32 = dict(device=DEV, dtype=torch.float32)
    outs = [torch.empty(513, **f32) for _ in range(5)]
    ws = torch.empty(lib.lce_forward_workspace_bytes(513, 256, 3000, 0), dtype=torch.uint8, device=DEV)
    args = lambda T: (h.data_ptr(), 256, w.data_ptr(), 256, y.data_ptr(), T, 256, 3000, 0, 1.0, 0,
                      *[o.data_ptr() for o in outs], ws.data_ptr(), ws.numel())
    assert lib.lce_forward_keep_logits(*args(513), buf.data_ptr(), buf.numel(), None) == -1
    assert lib.lce_forward_keep_logits(*args(64), buf.data_ptr(), 1000, None) == -2
    torch.cuda.synchronize()


def test_keep_logits_option_switches_the_autograd_node_to_recomputing():
    """LCE_OPT_KEEP_LOGITS_TOKENS = 0: no cache is offered, linear_cross_entropy's backward recomputes its logits, and
    the gradients are the same bits as with the logits kept."""
    from verl_amd import _abi, linear_cross_entropy
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    h, w, y, g_lp, g_ent = _case(96, 512, 30011, torch.bfloat16, seed=5)
    grads = []
    try:
        for tokens in (None, 0, 64):
            kernels.set_keep_logits_tokens(tokens)
            assert (lib.lce_logits_cache_bytes(96, 512, 30011, 0) > 0) == (tokens is None or tokens >= 96)
            hh, ww = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
            lp, ent = linear_cross_entropy(hh, ww, y, 0.9, "none")
            torch.autograd.backward([lp, ent], [g_lp, g_ent])
            grads.append((hh.grad, ww.grad))
        assert lib.lce_set_option(11, -1) != 0
    finally:
        kernels.set_keep_logits_tokens(None)
    for dh, dw in grads[1:]:
        assert torch.equal(dh, grads[0][0]) and torch.equal(dw, grads[0][1])


def test_kept_logits_are_bounded_in_aggregate():
    """A graph that holds several forwards at once (a long batch cut into pieces) keeps logits for at most as many rows
    in all as one call may keep (half the hidden size: 512 here): the third piece of 256 tokens keeps none and its
    backward recomputes, with the same gradients."""
    import gc

    import importlib

    from verl_amd import linear_cross_entropy

    mod = importlib.import_module("verl_amd.utils.kernel.linear_cross_entropy")  # (the package exports the function under this name)
    H, V = 1024, 5003
    row = (V + 63) // 64 * 64 * 4
    gc.collect()
    base = mod.kept_logits_bytes(DEV)
    pieces, outs = [], []
    w = (torch.randn(V, H) * 0.05).bfloat16().to(DEV).requires_grad_(True)
    for k in range(3):
        h, _, y, g_lp, g_ent = _case(256, H, V, torch.bfloat16, seed=20 + k)
        hh = h.clone().requires_grad_(True)
        lp, ent = linear_cross_entropy(hh, w, y, 1.0, "none")
        pieces.append((h, hh, y, g_lp, g_ent))
        outs.append((lp, ent))
        assert mod.kept_logits_bytes(DEV) - base == min(k + 1, 2) * 256 * row
    loss = sum((lp * p[3]).sum() + (ent * p[4]).sum() for (lp, ent), p in zip(outs, pieces))
    loss.backward()
    del outs, loss, lp, ent
    gc.collect()
    assert mod.kept_logits_bytes(DEV) == base
    dw = torch.zeros_like(w, dtype=torch.float32)
    for h, hh, y, g_lp, g_ent in pieces:
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w.detach(), y, 1.0)
        _bar(hh.grad, rdh)
        dw += rdw.float()
    err = (w.grad.float() - dw).abs()
    assert (err <= 3 * 2e-2 + 2.0**-6 * dw.abs()).all()  # three 16-bit gradients added by autograd


def test_few_token_step_replays_from_a_graph():
    """Forward (keeping its logits) and backward of a 64-token step recorded into a HIP graph: kernels only, no memset
    nodes.  Every replay, with new values in the same buffers (another set of tokens without gradient each time, so the
    token list built on the device changes) and eager work in between, must equal the eager calls on those inputs."""
    from verl_amd.utils.kernel import kernels

    T, H, V, tau = 64, 512, 20011, 0.9
    h, w, y, g_lp, g_ent = _case(T, H, V, torch.bfloat16, seed=31)

    def step():
        lp, ent, mx, acc, eb, cache = kernels.forward_keeping_logits(h, w, y, 0, tau)
        assert cache is not None
        dh, dw = kernels.efficient_entropy_backward(g_lp, g_ent, h, w, y, mx, acc, eb, 0, False, tau, logits_cache=cache)
        return lp, ent, dh, dw

    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        outs = step()
    for rep in range(3):
        h.copy_(((torch.rand(T, H) - 0.5) * (rep + 1)).bfloat16())
        y.copy_(torch.randint(0, V, (T,)))
        g_lp.copy_(torch.randn(T))
        g_ent.copy_(torch.randn(T))
        g_lp[rep::3] = 0.0
        g_ent[rep::3] = 0.0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = step()
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), (rep, (a.float() - b.float()).abs().max().item())
