"""lce_forward_static (the forward on the library's built-in scratch buffer, no allocation, no caller workspace)
against lce_forward through the C ABI: two calls in a row, the second on a smaller input, each bit-identical to the
workspace version; the size limit; that a call allocates no device memory; a captured and replayed call; and the
refusal of a call that would race with one still running on another stream."""

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


def _static_call(lib, _abi, h, w, y, tau, outs, stream):
    T, H = h.shape
    return lib.lce_forward_static(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), T, H, w.shape[0], _abi.DTYPE_BF16, tau, 0,
                                  *[o.data_ptr() for o in outs], stream)


def test_static_scratch_forward_allocates_no_device_memory():
    """What the entry point exists for: with every output preallocated, a call (after the first one on the device, which
    looks the buffer up) leaves both the driver's free-memory figure and torch's allocator untouched."""
    from verl_amd import _abi

    lib = _abi.load()
    h, w, y = _inputs(3000, 256, 7001, 5)
    outs = [torch.empty(3000, device=DEV) for _ in range(5)]
    st = torch.cuda.current_stream().cuda_stream
    _abi.check(_static_call(lib, _abi, h, w, y, 1.0, outs, st), "first call")
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        _abi.check(_static_call(lib, _abi, h, w, y, 1.0, outs, st), "lce_forward_static")
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0


def test_static_scratch_forward_under_graph_capture_replays_correctly():
    """After one call outside a capture the entry point can be recorded into a HIP graph (it launches kernels only, no
    memset node, and nothing in the buffer has to start at zero).  Every replay, with eager work and
    synchronisations of the program in between, must equal the workspace forward on the inputs of that moment."""
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V, tau = 2000, 256, 9001, 0.8
    h, w, y = _inputs(T, H, V, 6)
    outs = [torch.full((T,), float("nan"), device=DEV) for _ in range(5)]
    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _abi.check(_static_call(lib, _abi, h, w, y, tau, outs, side.cuda_stream), "warm-up call")
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _abi.check(_static_call(lib, _abi, h, w, y, tau, outs, torch.cuda.current_stream().cuda_stream), "captured call")
    for rep in range(3):
        # new input values in the same buffers, eager work of the program, then the replay
        h.copy_(((torch.rand(T, H) - 0.5) * (rep + 1)).bfloat16())
        y.copy_(torch.randint(0, V, (T,)))
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = _forward(lib, _abi, h, w, y, tau, static=False)
        for a, b in zip(outs, want):
            assert torch.equal(a, b), (rep, (a - b).abs().max().item())


def test_static_scratch_forward_refuses_a_call_that_would_race():
    """All calls on a GPU share the one buffer.  A call on another stream while the previous one is still running gets
    LCE_E_BUSY (-4) and launches nothing; once the first stream has finished the same call goes through."""
    from verl_amd import _abi

    lib = _abi.load()
    T, H, V = 8192, 1024, 100_000  # some milliseconds of work: the second call arrives while it runs
    h, w, y = _inputs(T, H, V, 7)
    outs_a = [torch.empty(T, device=DEV) for _ in range(5)]
    outs_b = [torch.full((T,), float("nan"), device=DEV) for _ in range(5)]
    sa, sb = torch.cuda.Stream(device=DEV), torch.cuda.Stream(device=DEV)
    torch.cuda.synchronize()
    _abi.check(_static_call(lib, _abi, h, w, y, 1.0, outs_a, sa.cuda_stream), "call on stream a")
    rc = _static_call(lib, _abi, h, w, y, 1.0, outs_b, sb.cuda_stream)
    assert rc == -4, rc
    assert b"still running" in lib.lce_last_error()
    # the same stream may queue behind itself
    _abi.check(_static_call(lib, _abi, h, w, y, 1.0, outs_a, sa.cuda_stream), "second call on stream a")
    sa.synchronize()
    assert all(torch.isnan(o).all() for o in outs_b)  # the refused call wrote nothing
    _abi.check(_static_call(lib, _abi, h, w, y, 1.0, outs_b, sb.cuda_stream), "call on stream b after a has finished")
    sb.synchronize()
    for a, b in zip(outs_a, outs_b):
        assert torch.equal(a, b)
