"""Direct calls of the C ABI (no Python wrapper in between): row strides larger than H, a workspace
placed at an odd offset, error codes for bad arguments on the device, and a non-default stream."""

import pytest
import torch

from oracle import lce_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(lib, _abi, h, ldh, w, ldw, y, T, H, V, dtype, tau, g_lp, g_ent, stream, vchunk=0, ws_shift=0):
    code = _abi.dtype_code(dtype)
    f32 = dict(device=DEV, dtype=torch.float32)
    lp, ent, mx, acc, eb = (torch.empty(T, **f32) for _ in range(5))
    nf = lib.lce_forward_workspace_bytes(T, H, V, code)
    ws = torch.empty(nf + 256, device=DEV, dtype=torch.uint8)
    rc = lib.lce_forward(h.data_ptr(), ldh, w.data_ptr(), ldw, y.data_ptr(), T, H, V, code, tau, 0, lp.data_ptr(), ent.data_ptr(),
                         mx.data_ptr(), acc.data_ptr(), eb.data_ptr(), ws.data_ptr(), nf, stream)
    _abi.check(rc, "lce_forward")
    dh = torch.empty(T, H, device=DEV, dtype=dtype)
    dw = torch.empty(V, H, device=DEV, dtype=dtype)
    nb = lib.lce_backward_workspace_bytes(T, H, V, code, vchunk)
    wsb = torch.empty(nb + 512, device=DEV, dtype=torch.uint8)
    rc = lib.lce_backward(h.data_ptr(), ldh, w.data_ptr(), ldw, y.data_ptr(), T, H, V, code, tau, 0, mx.data_ptr(), acc.data_ptr(),
                          eb.data_ptr(), g_lp.data_ptr(), g_ent.data_ptr(), dh.data_ptr(), dw.data_ptr(),
                          wsb.data_ptr() + ws_shift, nb, vchunk, stream)
    _abi.check(rc, "lce_backward")
    return lp, ent, dh, dw


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_padded_row_strides_side_stream_and_shifted_workspace(dtype):
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V, tau = 333, 256, 3001, 0.7
    pad_h, pad_w = 64, 8
    g = torch.Generator().manual_seed(5)
    hbuf = (torch.rand(T, H + pad_h, generator=g) - 0.5).to(dtype).to(DEV)
    wbuf = (torch.rand(V, H + pad_w, generator=g) - 0.5).to(dtype).to(DEV)
    h, w = hbuf[:, :H], wbuf[:, :H]
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    g_lp = (torch.rand(T, generator=g) * 2 - 1).to(DEV)
    g_ent = (torch.rand(T, generator=g) - 0.5).to(DEV)
    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        lp, ent, dh, dw = _call(lib, _abi, hbuf, H + pad_h, wbuf, H + pad_w, y, T, H, V, dtype, tau, g_lp, g_ent, side.cuda_stream,
                                vchunk=1024, ws_shift=16)
    side.synchronize()
    if dtype == torch.float32:
        rlp, rent = O.lce_forward(h, w, y, tau, compute_dtype=torch.float64)
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau, compute_dtype=torch.float64)
        for got, want in ((lp, rlp), (ent, rent), (dh, rdh), (dw, rdw)):
            err = (got.double() - want).abs().max().item()
            assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())
    else:
        rlp, rent = O.lce_forward(h, w, y, tau)
        rdh, rdw = O.lce_backward(g_lp, g_ent, h, w, y, tau)
        torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
        torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
        torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)


@pytest.mark.parametrize("dtype,T", [(torch.bfloat16, 520), (torch.float32, 520), (torch.bfloat16, 4200)])  # 4200: the 16x16x32 tiles
def test_hidden_spanning_more_than_4_gib_runs_without_the_token_list(dtype, T):
    """The backward lists the tokens with gradient and gathers their rows of `hidden` with 32-bit byte offsets;
    when T * ldh * esize reaches 4 GiB it runs on all tokens in place instead.  A [T, H] view with an 8 MiB row
    stride takes that branch at small T; tokens without gradient must still come out as exact zeros."""
    from verl_amd import _abi

    lib = _abi.load()
    H, V, tau = 256, 1500, 1.3
    ld = (8 << 20) // torch.empty((), dtype=dtype).element_size() + 64
    assert T * ld * torch.empty((), dtype=dtype).element_size() >= 1 << 32
    g = torch.Generator().manual_seed(7)
    hbuf = torch.empty(T, ld, device=DEV, dtype=dtype)
    hbuf[:, :H] = (torch.rand(T, H, generator=g) - 0.5).to(dtype).to(DEV)
    h = hbuf[:, :H]
    w = (torch.rand(V, H, generator=g) - 0.5).to(dtype).to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    keep = (torch.rand(T, generator=g) < 0.5).to(DEV)
    g_lp = (torch.rand(T, generator=g) * 2 - 1).to(DEV) * keep
    g_ent = (torch.rand(T, generator=g) - 0.5).to(DEV) * keep
    st = _abi.current_stream(torch.device(DEV))
    lp, ent, dh, dw = _call(lib, _abi, hbuf, ld, w, H, y, T, H, V, dtype, tau, g_lp, g_ent, st)
    torch.cuda.synchronize()
    cd = torch.float64 if dtype == torch.float32 else torch.float32
    rlp, rent = O.lce_forward(h, w, y, tau, compute_dtype=cd)
    rdh, rdw = O.lce_backward(g_lp.to(cd), g_ent.to(cd), h, w, y, tau, compute_dtype=cd)
    if dtype == torch.float32:
        for got, want in ((lp, rlp), (ent, rent), (dh, rdh), (dw, rdw)):
            err = (got.double() - want).abs().max().item()
            assert err <= 1e-5 * want.abs().max().item(), (err, want.abs().max().item())
    else:
        torch.testing.assert_close(lp, rlp, atol=1e-3, rtol=2e-4)
        torch.testing.assert_close(ent, rent, atol=5e-3, rtol=5e-4)
        torch.testing.assert_close(dh.float(), rdh, atol=2e-2, rtol=4e-2)
        torch.testing.assert_close(dw.float(), rdw, atol=2e-2, rtol=4e-2)
    assert torch.count_nonzero(dh[~keep]) == 0


def test_error_codes_leave_the_device_untouched():
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V = 8, 128, 100
    h = torch.zeros(T, H, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(V, H, device=DEV, dtype=torch.bfloat16)
    y = torch.zeros(T, device=DEV, dtype=torch.int64)
    out = torch.full((5, T), 7.0, device=DEV)
    ws = torch.empty(lib.lce_forward_workspace_bytes(T, H, V, 0), device=DEV, dtype=torch.uint8)
    st = _abi.current_stream(torch.device(DEV))
    args = lambda **kw: [kw.get("h", h.data_ptr()), kw.get("ldh", H), w.data_ptr(), kw.get("ldw", H), y.data_ptr(), T, H, V, 0,
                         kw.get("tau", 1.0), kw.get("red", 0), out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(),
                         out[3].data_ptr(), out[4].data_ptr(), ws.data_ptr(), kw.get("nws", ws.numel()), st]
    assert lib.lce_forward(*args(ldh=H - 8)) == -1           # row stride shorter than a row
    assert lib.lce_forward(*args(ldw=H + 3)) == -1           # row stride not a multiple of 16 bytes
    assert lib.lce_forward(*args(h=h.data_ptr() + 2)) == -1  # misaligned pointer
    assert lib.lce_forward(*args(ldh=1 << 23)) == -1         # 256 rows would span 4 GiB
    assert lib.lce_forward(*args(tau=0.0)) == -1
    assert lib.lce_forward(*args(red=9)) == -1
    assert lib.lce_forward(*args(nws=16)) == -2              # workspace too small
    assert b"workspace" in lib.lce_last_error()
    torch.cuda.synchronize()
    assert (out == 7.0).all()
    assert lib.lce_forward(*args()) == 0
    torch.cuda.synchronize()
    assert not (out == 7.0).any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_sum_pi_squared_backward_with_and_without_the_saved_row_statistics(dtype):
    """lce_logits_sum_pi_squared_backward takes the rows' logsumexp and sum p^2 from the forward, or recomputes both when
    they are NULL; both ways must give autograd's gradient of the reference expression
    (verl/utils/torch_functional.py:687-703) on a padded row stride."""
    from verl_amd import _abi

    lib = _abi.load()
    R, V, ld = 9, 5003, 5016
    g = torch.Generator().manual_seed(3)
    buf = (torch.randn(R, ld, generator=g) * 2).to(dtype).to(DEV)
    z = buf[:, :V]
    up = torch.randn(R, generator=g).to(DEV)
    code = _abi.dtype_code(dtype)
    st = torch.cuda.current_stream().cuda_stream
    s = torch.empty(R, device=DEV)
    lse = torch.empty(R, device=DEV)
    _abi.check(lib.lce_logits_sum_pi_squared(buf.data_ptr(), ld, R, V, code, s.data_ptr(), lse.data_ptr(), st), "forward")
    torch.testing.assert_close(lse.double(), torch.logsumexp(z.double(), -1), atol=1e-5, rtol=1e-6)
    zz = z.double().requires_grad_(True)
    (want,) = torch.autograd.grad(O.sum_pi_squared_from_logits(zz, torch.float64), zz, up.double())
    for with_stats in (True, False):
        d = torch.full((R, ld), 7.0, device=DEV, dtype=dtype)
        rc = lib.lce_logits_sum_pi_squared_backward(buf.data_ptr(), ld, R, V, code, lse.data_ptr() if with_stats else None,
                                                    s.data_ptr() if with_stats else None, up.data_ptr(), d.data_ptr(), ld, st)
        _abi.check(rc, "backward")
        got = d[:, :V].double()
        if dtype == torch.float32:
            assert ((got - want).abs().max() / want.abs().max()).item() < 1e-5
        else:
            assert ((got - want).abs() <= 2e-2 + want.abs() * 2.0**-7).all()
        assert (d[:, V:] == 7.0).all()  # the padding of the rows is not written
    assert lib.lce_logits_sum_pi_squared_backward(buf.data_ptr(), ld, R, V, code, None, None, None, d.data_ptr(), ld, st) != 0


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
def test_diagnostic_gemms_match_torch(variant):
    """lce_gemm_nt / lce_gemm_tn (the mainloops on their own, which the benchmark's yardstick workload times) against
    torch.matmul in fp32 on bf16 operands, ragged M and N."""
    from verl_amd import _abi

    lib = _abi.load()
    M, N, K = 300, 520, 192
    g = torch.Generator().manual_seed(variant)
    A = (torch.randn(M, K, generator=g)).bfloat16().to(DEV)
    B = (torch.randn(N, K, generator=g)).bfloat16().to(DEV)
    st = torch.cuda.current_stream().cuda_stream
    C = torch.zeros(M, N, device=DEV)
    _abi.check(lib.lce_gemm_nt(A.data_ptr(), K, B.data_ptr(), K, C.data_ptr(), N, M, N, K, 0, variant, st), "lce_gemm_nt")
    want = A.float() @ B.float().t()
    torch.testing.assert_close(C, want, atol=1e-3, rtol=1e-4)
    # K-major operands, rows allocated in whole 256-column tiles
    At = torch.zeros(K, 512, device=DEV, dtype=torch.bfloat16)
    Bt = torch.zeros(K, 768, device=DEV, dtype=torch.bfloat16)
    At[:, :M] = A.t()
    Bt[:, :N] = B.t()
    C2 = torch.zeros(M, N, device=DEV)
    _abi.check(lib.lce_gemm_tn(At.data_ptr(), 512, Bt.data_ptr(), 768, C2.data_ptr(), N, M, N, K, variant, st), "lce_gemm_tn")
    torch.testing.assert_close(C2, want, atol=1e-3, rtol=1e-4)
