"""lce_forward_static (the forward on the library's built-in scratch buffer, no allocation, no caller workspace)
against lce_forward through the C ABI: two calls in a row, the second on a smaller input, each bit-identical to the
workspace version; and the size limit."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(T, H, V, seed):
    g = torch.Generator().manual_seed(seed)
    h = (torch.rand(T, H, generator=g) - 0.5).bfloat16().to(DEV)
    w = (torch.rand(V, H, generator=g) - 0.5).bfloat16().to(DEV)
    y = torch.randint(0, V, (T,), generator=g).to(DEV)
    return h, w, y


def _forward(lib, _abi, h, w, y, tau, static):
    T, H = h.shape
    V = w.shape[0]
    f32 = dict(device=DEV, dtype=torch.float32)
    outs = [torch.full((T,), float("nan"), **f32) for _ in range(5)]
    st = torch.cuda.current_stream().cuda_stream
    if static:
        rc = lib.lce_forward_static(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), T, H, V, _abi.DTYPE_BF16, tau, 0,
                                    *[o.data_ptr() for o in outs], st)
        _abi.check(rc, "lce_forward_static")
    else:
        n = lib.lce_forward_workspace_bytes(T, H, V, _abi.DTYPE_BF16)
        ws = torch.empty(n, device=DEV, dtype=torch.uint8)
        rc = lib.lce_forward(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), T, H, V, _abi.DTYPE_BF16, tau, 0,
                             *[o.data_ptr() for o in outs], ws.data_ptr(), n, st)
        _abi.check(rc, "lce_forward")
    torch.cuda.synchronize()
    return outs


def test_static_scratch_forward_matches_workspace_forward_twice_in_a_row():
    from verl_amd import _abi

    lib = _abi.load()
    tau = 1.3
    # the second call is smaller in every dimension (fewer tokens: other split count and tile shape; smaller vocabulary)
    for T, H, V, seed in ((9000, 256, 5003, 1), (700, 128, 1001, 2)):
        h, w, y = _inputs(T, H, V, seed)
        got = _forward(lib, _abi, h, w, y, tau, static=True)
        want = _forward(lib, _abi, h, w, y, tau, static=False)
        for a, b in zip(got, want):
            assert torch.equal(a, b), (T, (a - b).abs().max().item())
        assert torch.isfinite(got[0]).all() and torch.isfinite(got[1]).all()


def test_static_scratch_forward_where_the_buffer_limits_the_split_count():
    """13312 tokens against 152064 vocabulary rows: the workspace forward cuts the vocabulary into 54 splits (11.5 MB of
    partial statistics), the 8 MiB buffer has room for 39.  Another partition of the same fp32 sums: equal to 1e-5
    (relative to the largest value), not bit for bit."""
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V = 13312, 128, 152064
    assert lib.lce_forward_workspace_bytes(T, H, V, _abi.DTYPE_BF16) > (8 << 20)
    h, w, y = _inputs(T, H, V, 3)
    got = _forward(lib, _abi, h, w, y, 0.9, static=True)
    want = _forward(lib, _abi, h, w, y, 0.9, static=False)
    for a, b in zip(got, want):
        assert torch.isfinite(a).all()
        assert (a - b).abs().max().item() <= 1e-5 * max(1.0, b.abs().max().item())


def test_static_scratch_forward_rejects_sizes_beyond_its_buffer():
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V = 200_000, 128, 512
    z = torch.zeros(1, device=DEV)
    rc = lib.lce_forward_static(z.data_ptr(), H, z.data_ptr(), H, z.data_ptr(), T, H, V, _abi.DTYPE_BF16, 1.0, 0, z.data_ptr(),
                                z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), None)
    assert rc == -2
    assert b"lce_forward_static" in lib.lce_last_error()
