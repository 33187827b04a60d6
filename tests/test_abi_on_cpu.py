"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol the
header declares, and the Python surface rejects bad arguments the way the reference does
(verl/utils/kernel/linear_cross_entropy.py:64-65, verl/utils/kernel/kernels.py:113-126)."""

import ctypes
import inspect
import os
import re

import pytest
import torch

from verl_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_functions():
    text = open(os.path.join(ROOT, "include", "lce_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lce_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _header_functions()
    assert len(names) >= 12
    lib = ctypes.CDLL(_abi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/lce_abi.h but not exported"
    assert sorted(_abi.SYMBOLS) == names, "python binding and header disagree"


def test_abi_version_and_error_string():
    lib = _abi.load()
    assert lib.lce_abi_version() == _abi.ABI_VERSION
    assert lib.lce_num_variants() >= 1
    assert lib.lce_set_variant(10_000) != 0
    assert b"variant" in lib.lce_last_error()
    # argument validation happens before any device work
    rc = lib.lce_forward(None, 128, None, 128, None, 4, 100, 10, 0, 1.0, 0, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"multiple of 64" in lib.lce_last_error()
    rc = lib.lce_forward(None, 128, None, 128, None, 4, 128, 10, 7, 1.0, 0, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"dtype" in lib.lce_last_error()
    assert lib.lce_forward_workspace_bytes(16384, 3584, 152064, 0) < (64 << 20)
    # backward workspace stays far below a [T, V] tile pair: bounded d_logits chunk + transposed operands + fp32 d_hidden
    # (at every token count: few tokens add K-split partials of d_hidden, many tokens narrow the chunk)
    for T, H, V, dt in [(16384, 3584, 152064, 0), (8192, 2048, 152064, 0), (64, 3584, 152064, 0), (1024, 4096, 128256, 0),
                        (4096, 3584, 152064, 1), (65536, 5120, 152064, 0), (262144, 4096, 128256, 0)]:
        esz = 2 if dt == 0 else 4
        assert lib.lce_backward_workspace_bytes(T, H, V, dt, 0) < 0.25 * T * V * esz + 4 * V * H, (T, H, V, dt)


def test_default_chunk_rule_and_workspace_budget():
    """Default: chunks of 16384 vocabulary columns (wider while one d_logits buffer stays within 256 MiB; from 8192 columns
    on while one stays within 1 GiB; narrower once two of them would pass 4 GiB), so the backward's workspace at config 2
    is under 1.5 GiB; a byte budget (kernels.set_workspace_budget / LCE_OPT_WORKSPACE_BUDGET) makes
    the library pick the widest chunk that fits, never exceeding its upper bound and never going below 2048 columns; an
    explicit chunk width wins over both."""
    from verl_amd.utils.kernel import kernels

    lib = _abi.load()
    T, H, V = 16384, 3584, 152064
    gate = 0.25 * T * V * 2 + 4 * V * H
    try:
        default = lib.lce_backward_workspace_bytes(T, H, V, 0, 0)
        assert default < (3 << 29)
        assert lib.lce_backward_workspace_bytes(T, H, V, 0, 15360) == default  # the 10 chunks that 16384 columns need, evened out
        # few tokens: the whole vocabulary in one chunk (one single-buffered d_logits tile)
        few = lib.lce_backward_workspace_bytes(64, H, V, 0, 0)
        assert few == lib.lce_backward_workspace_bytes(64, H, V, 0, 152064)
        # very many tokens: narrower chunks, so that the two d_logits buffers stay within 4 GiB
        assert lib.lce_backward_workspace_bytes(65536, 5120, V, 0, 0) == lib.lce_backward_workspace_bytes(65536, 5120, V, 0, 8192)
        assert lib.lce_backward_workspace_bytes(262144, 4096, 128256, 0, 0) == lib.lce_backward_workspace_bytes(262144, 4096, 128256, 0, 4096)
        assert lib.lce_backward_workspace_bytes(1 << 21, 4096, 128256, 0, 0) == lib.lce_backward_workspace_bytes(1 << 21, 4096, 128256, 0, 2048)
        sizes = []
        for budget in (600 << 20, 1 << 30, 5 << 29, 1 << 40):
            kernels.set_workspace_budget(budget)
            n = lib.lce_backward_workspace_bytes(T, H, V, 0, 0)
            sizes.append(n)
            assert n < gate
            if budget >= (700 << 20):
                assert n <= min(budget, gate)
        assert sizes == sorted(sizes) and sizes[0] < default < sizes[2] and sizes[3] > (2 << 30)
        # a budget no chunk of at least 2048 columns fits: the floor is what is reported (and what lce_backward asks for)
        kernels.set_workspace_budget(1 << 20)
        assert lib.lce_backward_workspace_bytes(T, H, V, 0, 0) == lib.lce_backward_workspace_bytes(T, H, V, 0, 2048)
        # an explicit width is not touched by the budget
        assert lib.lce_backward_workspace_bytes(T, H, V, 0, 15360) == default
    finally:
        kernels.set_workspace_budget(0)
    assert lib.lce_backward_workspace_bytes(T, H, V, 0, 0) == default
    assert lib.lce_set_option(8, -1) != 0


def test_signature_matches_reference():
    from verl_amd.utils.kernel.linear_cross_entropy import LinearCrossEntropy
    from verl_amd.utils.kernel import kernels

    sig = inspect.signature(LinearCrossEntropy.forward)
    assert list(sig.parameters) == ["ctx", "hidden", "weight", "labels", "temperature", "reduction", "dist_process_group"]
    assert sig.parameters["temperature"].default == 1.0 and sig.parameters["reduction"].default == "none"
    fsig = inspect.signature(kernels.efficient_entropy_forward)
    assert list(fsig.parameters) == ["hidden", "weight", "labels", "reduction", "temperature", "dist_process_group"]
    bsig = inspect.signature(kernels.efficient_entropy_backward)
    positional = [n for n, p in bsig.parameters.items() if p.kind is not inspect.Parameter.KEYWORD_ONLY]
    assert positional == [
        "dlogprobs", "dentropy", "hidden", "weight", "labels", "maximum", "acc", "entropy_b", "reduction",
        "should_return_fp32_grad", "temperature", "dist_process_group",
    ]  # fmt: skip
    # beyond the reference's: keyword-only arguments that default to the reference's behaviour (both gradients, the
    # logits recomputed)
    extras = {n: p.default for n, p in bsig.parameters.items() if p.kind is inspect.Parameter.KEYWORD_ONLY}
    assert extras == {"need_d_hidden": True, "need_d_weight": True, "logits_cache": None}
    assert kernels.get_entropy_reduction_enum_number("none") == 0
    assert kernels.get_entropy_reduction_enum_number("sum") == 1
    assert kernels.get_entropy_reduction_enum_number("mean") == 2
    with pytest.raises(ValueError, match="Invalid reduction"):
        kernels.get_entropy_reduction_enum_number("max")
    kernels.set_backward_method(kernels.BackwardEnum._Total_Separate)
    kernels.set_backward_method(kernels.BackwardEnum._Split_Dlogits_N)


def test_argument_errors_before_device_work():
    from verl_amd import linear_cross_entropy

    h = torch.zeros(4, 128)
    w = torch.zeros(16, 128)
    y = torch.zeros(4, dtype=torch.long)
    with pytest.raises(AssertionError, match="temperature must be a float"):
        linear_cross_entropy(h, w, y, 1, "none")
    with pytest.raises(AssertionError, match="reduction must be a str"):
        linear_cross_entropy(h, w, y, 1.0, None)
    with pytest.raises(ValueError, match="Invalid reduction"):
        linear_cross_entropy(h, w, y, 1.0, "max")
    with pytest.raises(AssertionError):  # CPU tensors: the reference asserts is_cuda
        linear_cross_entropy(h, w, y, 1.0, "none")


def test_no_fallback_when_library_is_missing(monkeypatch, tmp_path):
    monkeypatch.setattr(_abi, "_lib", None)
    monkeypatch.setattr(_abi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_abi.LceError, match="no CPU or eager fallback"):
        _abi.load()


def test_product_code_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "verl_amd")
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(d, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


def test_fused_linear_for_ppo_constructor():
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO

    with pytest.raises(ValueError, match="Unsupported FusedLinearForPPO backend"):  # tests/utils/test_experimental_torch_functional_on_cpu.py:127-129
        FusedLinearForPPO(impl_backend="nope")
    m = FusedLinearForPPO(chunk_size=3)
    with pytest.raises(ValueError):
        m(torch.zeros(2, 3, 4, 8), torch.zeros(5, 8), torch.zeros(2, 3, 4, dtype=torch.long))


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more exits with a message instead of pretending."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr


def test_process_group_of_one_rank_is_the_single_gpu_path():
    """Megatron hands its tensor-parallel group over even at size 1 (verl/models/mcore/model_forward_fused.py:110-117)."""
    import torch.distributed as dist

    from verl_amd.utils.kernel.kernels import _require_single_rank

    class Two:
        def size(self):
            return 2

    _require_single_rank(None)
    with pytest.raises(NotImplementedError):
        _require_single_rank(Two())
    with pytest.raises(NotImplementedError):
        _require_single_rank(object())
    created = not dist.is_initialized()
    if created:
        dist.init_process_group("gloo", init_method="tcp://127.0.0.1:29531", rank=0, world_size=1)
    try:
        _require_single_rank(dist.group.WORLD)
        _require_single_rank(dist.new_group([0]))
    finally:
        if created:
            dist.destroy_process_group()


def test_logits_twins_name_the_gpu_only_precondition():
    """The reference's twins run on any device (its own CPU tests call them); these are HIP kernels without a fallback
    and say so with a named error instead of a bare assert."""
    from verl_amd.utils import torch_functional as F

    z = torch.zeros(2, 8)
    for call in (lambda: F.entropy_from_logits(z), lambda: F.logprobs_from_logits(z, torch.zeros(2, dtype=torch.long)),
                 lambda: F.calculate_sum_pi_squared_from_logits(z)):
        with pytest.raises(_abi.LceError, match="GPU tensors only"):
            call()


def test_metric_aggregation_kinds_of_ppo_loss():
    """verl/workers/utils/losses.py:71-84: any global normaliser switches the loss metrics to SUM; Metric folds as
    verl/utils/metric/utils.py:72-160 (hand-computed numbers)."""
    from verl_amd.trainer.ppo import core_algos as C
    from verl_amd.utils.metric import AggregationType, Metric
    from verl_amd.workers.utils.losses import metric_aggregation_for

    assert metric_aggregation_for(1, None, None, None) == AggregationType.MEAN
    assert metric_aggregation_for(2, None, None, None) == AggregationType.SUM
    assert metric_aggregation_for(1, 100, None, None) == AggregationType.SUM
    assert metric_aggregation_for(1, None, 8, None) == AggregationType.SUM
    assert metric_aggregation_for(1, None, None, 512) == AggregationType.SUM
    m = Metric("mean", 1.0)
    m.append(torch.tensor(2.0))
    m.append(Metric(AggregationType.MEAN, [3.0, 6.0]))
    assert m.aggregate() == 3.0
    assert Metric("sum", [1, 2, 3.5]).aggregate() == 6.5
    assert Metric("min", [4, 2, 3]).aggregate() == 2 and Metric("max", [4, 2, 3]).aggregate() == 4
    with pytest.raises(ValueError, match="mismatch"):
        m.append(Metric("sum", 1.0))
    with pytest.raises(ValueError, match="scalar"):
        m.append(torch.zeros(2))
    with pytest.raises(ValueError):
        Metric("median")
    # two ranks, two accumulation steps: SUM adds the per-step means over ranks, MAX looks at every value
    assert Metric.aggregate_dp([Metric("sum", [1.0, 3.0]), Metric("sum", [3.0, 5.0])]) == 6.0
    assert Metric.aggregate_dp([Metric("mean", [1.0, 3.0]), Metric("mean", [3.0, 5.0])]) == 3.0
    assert Metric.aggregate_dp([Metric("max", [1.0, 9.0]), Metric("max", [3.0, 5.0])]) == 9.0
    with pytest.raises(ValueError, match="same number of values"):
        Metric.aggregate_dp([Metric("sum", [1.0]), Metric("sum", [1.0, 2.0])])
    d = Metric.from_dict({"a": 1.0, "b": 2.0}, "mean")
    assert d["b"].aggregate() == 2.0 and d["a"].aggregation == AggregationType.MEAN
    with pytest.raises(ValueError, match="Unsupported loss mode: gpg"):
        C.get_policy_loss_fn("gpg")


def test_metric_values_are_plain_numbers_for_every_consumer():
    """verl/utils/metric/utils.py:103-113 turns an appended tensor into a float at once; here the read-back is deferred
    until somebody looks, and from then on `values`, a pickle, `repr`, `init_list` and `reduce_metrics` (:25-58, :162-163)
    see what the reference's consumers see: floats, never tensors."""
    import pickle

    from verl_amd.utils.metric import AggregationType, Metric, reduce_metrics

    m = Metric("mean", torch.tensor(1.5))
    m.append(torch.tensor([2.5]))
    m.append(4)
    assert any(isinstance(v, torch.Tensor) for v in m._items)  # nothing has been read back yet
    twin = pickle.loads(pickle.dumps(m))
    assert twin.values == [1.5, 2.5, 4] and all(not isinstance(v, torch.Tensor) for v in twin.values)
    assert twin.aggregation == AggregationType.MEAN and twin.aggregate() == pytest.approx(8.0 / 3)
    assert m.values == [1.5, 2.5, 4] and all(isinstance(v, (int, float)) for v in m.values)
    assert not any(isinstance(v, torch.Tensor) for v in m._items)  # read back once, kept as floats
    assert "tensor" not in repr(m)
    e = m.init_list()
    assert e.values == [] and e.aggregation == AggregationType.MEAN
    # extending from a metric with pending scalars keeps them pending, and folds the same
    a = Metric("sum", torch.tensor(2.0))
    b = Metric("sum", [1.0])
    b.extend(a)
    assert b.aggregate() == 3.0
    out = reduce_metrics({"actor/pg_loss": Metric("sum", [1.0, 2.0]), "x_max": [1.0, 5.0], "x_min": [1.0, 5.0], "y": [1.0, 5.0]})
    assert out == {"actor/pg_loss": 3.0, "x_max": 5.0, "x_min": 1.0, "y": 3.0}
    m.values = [7.0, torch.tensor(9.0)]
    assert m.values == [7.0, 9.0]


def test_tile_map_covers_every_tile_once_and_balances_the_xcds(tmp_path):
    """The workgroup -> tile map of all tiled kernels, checked exhaustively on the host (tests/tile_map_check.cpp):
    a hole or a duplicate would be a wrong result on the GPU, an uneven split over the 8 XCDs a slow one (a forward with
    12 token tiles x 20 splits used to leave one XCD with 40 of the 240 workgroups and take two rounds)."""
    import subprocess

    here = os.path.dirname(os.path.abspath(__file__))
    exe = str(tmp_path / "tile_map_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-o", exe, os.path.join(here, "tile_map_check.cpp")], check=True, timeout=300)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.startswith("ok"), r.stdout + r.stderr
