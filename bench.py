"""Headline benchmark: fwd+bwd tokens/s of the fused lm-head log-prob + entropy at a Qwen2.5-7B-shaped head.

One "step" = linear_cross_entropy forward + backward over one synthetic micro-batch that is
already resident in HBM (T=16384, H=3584, V=152064, bf16, temperature 1.0, upstream grads ~N(0,1)).
Prints ONE JSON line with the throughput, the roofline of the dominant kernel (HIP-event timed in
this run) and the CPU baseline (the oracle's torch restatement on the host cores, bounded sample).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16 = 2500e12  # MI355X dense bf16 MFMA peak, FLOP/s
# HBM-side bytes per launch (fetch + write) of the dominant kernels come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# (counters cannot be read from inside this process) and are kept in profiles/traffic.json together with the library state
# they were measured at; a run whose state differs reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def library_state(lib, T, H, V, flags):
    """What decides the tiling of a run: ABI version, the workspace sizes the library derives for this shape (they move
    with the mainloop variant, the chunk width and the layout options) and the tuning flags given on the command line."""
    return {
        "abi": int(lib.lce_abi_version()),
        "forward_workspace_bytes": int(lib.lce_forward_workspace_bytes(T, H, V, 0)),
        "backward_workspace_bytes": int(lib.lce_backward_workspace_bytes(T, H, V, 0, 0)),
        "flags": flags,
    }


def measured_traffic(workload, kernel, state):
    try:
        table = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return None
    rec = table.get(workload, {}).get(kernel)
    if not rec or rec.get("state") != state:
        return None
    return rec.get("bytes_per_launch")


WORKLOADS = {
    # name: (T, H, V, temperature, weight std, sequences, shortest valid length, PPO loss in the step[, forward only])
    # `sequences` > 0: T is that many equally long rows, each with a valid prefix of U{shortest..row}
    # tokens; the upstream gradients are zero on the masked suffix (as a PPO response mask gives them).
    "qwen2.5-7b-head-T16384": (16384, 3584, 152064, 1.0, 0.02, 0, 0, False),
    "llama3-8b-head-T32768": (32768, 4096, 128256, 0.6, 0.02, 8, 512, False),
    "qwen2.5-32b-head-T65536": (65536, 5120, 152064, 1.0, 0.015, 0, 0, False),
    # one actor micro-step: forward, clipped PPO loss (eps 0.2, dual clip 3.0, token-mean) with entropy
    # bonus 1e-3, backward; the loss kernel produces the upstream gradients
    "llama3-8b-actor-step-T262144": (262144, 4096, 128256, 1.0, 0.02, 64, 256, True),
    # log-prob pass with few tokens: one streaming read of W, HBM-bound
    "qwen2.5-7b-head-T64-fwd": (64, 3584, 152064, 1.0, 0.02, 0, 0, False, True),
    # few tokens, forward + backward: every kernel streams W (or writes d_weight) once, HBM-bound
    "qwen2.5-7b-head-T64": (64, 3584, 152064, 1.0, 0.02, 0, 0, False),
    # the log-prob passes that run under no_grad (old_log_prob, ref_log_prob): forward only at the full token count
    "qwen2.5-7b-head-T16384-fwd": (16384, 3584, 152064, 1.0, 0.02, 0, 0, False, True),
    "small": (2048, 1024, 32768, 1.0, 0.02, 0, 0, False),
}


def cpu_model_name() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(seconds_budget: float = 20.0):
    """The oracle's torch restatement (materialised fp32 logits) on the host cores: forward on the
    CPU-runnable reference case (T=1024, H=896, V=151936), bounded to a sample of rows sized so the
    whole leg takes about `seconds_budget`: one warm-up, then the median of five runs; reported in tokens/s."""
    import torch

    from oracle import lce_oracle as O

    cores = os.cpu_count() or 1
    # respect the box's CPU share if it is advertised
    for var in ("OMP_NUM_THREADS", "MAX_JOBS"):
        if os.environ.get(var, "").isdigit():
            cores = min(cores, int(os.environ[var]))
            break
    torch.set_num_threads(cores)
    T, H, V = 1024, 896, 151936
    g = torch.Generator().manual_seed(1235)
    h = torch.randn(T, H, generator=g)
    w = torch.randn(V, H, generator=g) * 0.02
    y = torch.randint(0, V, (T,), generator=g)
    rows = 128
    t0 = time.perf_counter()
    O.lce_forward(h[:rows], w, y[:rows], 1.0, chunk=128)  # sizes the sample
    dt = time.perf_counter() - t0
    runs = 5
    rows = int(max(128, min(T, rows * (seconds_budget / (runs + 1.0)) / max(dt, 1e-3))))
    rows = (rows // 128) * 128
    O.lce_forward(h[:rows], w, y[:rows], 1.0, chunk=128)  # warm-up at the sample size
    times = []
    for _ in range(runs):
        t0 = time.perf_counter()
        O.lce_forward(h[:rows], w, y[:rows], 1.0, chunk=128)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[runs // 2]
    return {
        "value": rows / med,
        "unit": "tokens/s (forward only, fp32)",
        "cores": cores,
        "torch_num_threads": torch.get_num_threads(),
        "cpu_model": cpu_model_name(),
        "kind": "port",
        "sample": f"oracle torch restatement, forward, first {rows} of T=1024 rows, H=896, V=151936, fp32, 1 warm-up + median of {runs}",
        "runs_s": [round(t, 4) for t in times],
        "gflops": 2.0 * rows * H * V / med / 1e9,
    }


def unfused_context(h, w, y, tau, g_lp, g_ent):
    """Forward + backward of the oracle's autograd restatement (`oracle.lce_oracle.lce_unfused_autograd`: one fp32
    [T, V] logits tensor) on the GPU: milliseconds and peak extra device memory.  Any failure (memory) is reported, not raised."""
    import torch

    from oracle import lce_oracle as O

    dev = h.device
    try:
        out = None
        for _ in range(2):  # warm-up (hipBLASLt heuristics, allocator), then the timed run
            del out
            torch.cuda.synchronize()
            base = torch.cuda.memory_allocated(dev)
            torch.cuda.reset_peak_memory_stats(dev)
            t0 = time.perf_counter()
            out = O.lce_unfused_autograd(h, w, y, tau, g_lp, g_ent, torch.float32)
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3
            peak = torch.cuda.max_memory_allocated(dev) - base
        del out
        torch.cuda.empty_cache()
        return {"what": "reference test's torch path: fp32 [T, V] logits materialised, softmax + logsumexp + cross_entropy, autograd",
                "fwd_bwd_ms": ms, "peak_extra_bytes": peak}
    except Exception as e:  # noqa: BLE001
        torch.cuda.empty_cache()
        return {"error": f"{type(e).__name__}: {str(e)[:200]}"}


PEAK_HBM = 8e12  # MI355X HBM3E peak, bytes/s

LOGITS_WORKLOADS = {
    # name: (rows, vocabulary): logits that already exist in HBM, bf16
    "logits-twins-R8192-V152064": (8192, 152064),
    # the same through logprobs_and_entropy_from_logits: one forward pass, one backward pass, one d_logits
    "logits-twins-combined-R8192-V152064": (8192, 152064, True),
}


def run_logits_workload(args, name):
    """The unfused twins on given logits (logprobs_from_logits + entropy_from_logits): HBM-bound row
    reductions; one step = both forward passes and both backward passes over one [R, V] bf16 tensor."""
    import torch

    from verl_amd import _abi
    from verl_amd.utils import torch_functional as F

    lib = _abi.load()
    state = {"abi": int(lib.lce_abi_version())}  # (these kernels have no workspace and no tuning flags)
    if args.print_state:
        print(json.dumps({"workload": name, "state": state}), flush=True)
        return
    dev = torch.device("cuda:0")
    R, V = LOGITS_WORKLOADS[name][:2]
    combined = len(LOGITS_WORKLOADS[name]) > 2 and LOGITS_WORKLOADS[name][2]
    g = torch.Generator(device=dev).manual_seed(1234 + 6)
    z = (torch.randn(R, V, device=dev, generator=g) * 3).bfloat16().requires_grad_(True)
    y = torch.randint(0, V, (R,), device=dev, generator=g)
    if args.copy_calibration:
        src = torch.empty(1 << 30, device=dev, dtype=torch.uint8).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 1 GiB, writes 1 GiB per launch
        torch.cuda.synchronize()
        del src, dst
    g_lp = torch.randn(R, device=dev, generator=g).bfloat16()
    g_ent = torch.randn(R, device=dev, generator=g).bfloat16()

    def step():
        z.grad = None
        if combined:
            lp, ent = F.logprobs_and_entropy_from_logits(z, y)
        else:
            lp = F.logprobs_from_logits(z, y)
            ent = F.entropy_from_logits(z)
        torch.autograd.backward([lp, ent], [g_lp, g_ent])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.lce_profile_enable(1)
    _abi.profile_read(reset=True)
    nprof = max(2, min(args.steps, 5))
    for _ in range(nprof):
        step()
    torch.cuda.synchronize()
    prof = _abi.profile_read(reset=True)
    lib.lce_profile_enable(0)
    kernels = {k: {"ms_per_step": ms / nprof, "launches_per_step": n / nprof, "avg_ms": ms / n} for k, (ms, n) in prof.items()}
    # algorithmic bytes per launch: forward reads the logits once; backward reads them once and writes d_logits once
    bytes_per_launch = {"logits_fwd_kernel": R * V * 2.0, "logits_bwd_kernel": 2.0 * R * V * 2.0}
    for k, v in kernels.items():
        if k in bytes_per_launch:
            v["achieved_GBps"] = bytes_per_launch[k] / (v["avg_ms"] * 1e-3) / 1e9
    dom = max((k for k in kernels if k in bytes_per_launch), key=lambda k: kernels[k]["ms_per_step"])
    achieved = bytes_per_launch[dom] / (kernels[dom]["avg_ms"] * 1e-3)
    out = {
        "metric": "rows/s, logprobs_from_logits + entropy_from_logits forward and backward on given logits",
        "value": R / (elapsed / args.steps),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": name, "R": R, "V": V, "pass": "1 x fwd + 1 x bwd (one autograd node)" if combined else "2 x fwd + 2 x bwd (+ torch's accumulation of the two d_logits)"},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved / 1e9, "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": achieved / PEAK_HBM, "traffic": measured_traffic(name, dom, state), "avg_launch_ms": kernels[dom]["avg_ms"],
                     "bytes_per_launch": bytes_per_launch[dom]},
        "kernels": kernels,
        "cpu_baseline": None,
    }
    print(json.dumps(out), flush=True)


CEILING_WORKLOAD = "mfma-ceiling"


class _PowerSampler:
    """Socket power (W) and shader clock (MHz) of GPU 0 sampled every 50 ms through amdsmi on a host thread; every
    reading is None where the module or a field is missing."""

    def __init__(self):
        import threading

        self.samples = []
        self._stop = False
        self.error = None
        self._thread = threading.Thread(target=self._run, daemon=True)
        self._thread.start()

    def _run(self):
        try:
            try:
                import amdsmi
            except ImportError:
                sys.path.insert(0, "/opt/rocm/share/amd_smi")
                import amdsmi
            amdsmi.amdsmi_init()
            handle = amdsmi.amdsmi_get_processor_handles()[0]
            try:
                self.cap_watts = amdsmi.amdsmi_get_power_cap_info(handle).get("power_cap", 0) / 1e6
            except Exception:
                self.cap_watts = None
            while not self._stop:
                p = amdsmi.amdsmi_get_power_info(handle)
                c = amdsmi.amdsmi_get_clock_info(handle, amdsmi.AmdSmiClkType.GFX)
                watts = p.get("current_socket_power", p.get("average_socket_power"))
                mhz = c.get("clk", c.get("cur_clk"))
                self.samples.append((time.time(), watts if isinstance(watts, (int, float)) else None, mhz if isinstance(mhz, (int, float)) else None))
                time.sleep(0.05)
        except Exception as e:  # no amdsmi, no permission: the rates are still measured
            self.error = f"{type(e).__name__}: {e}"

    def window(self, t0, t1):
        """Mean power and clock over the last 60 % of [t0, t1] (the governor has settled by then)."""
        ta = t0 + 0.4 * (t1 - t0)
        sel = [(w, c) for (t, w, c) in self.samples if ta <= t <= t1]
        ws = [w for w, _ in sel if w is not None]
        cs = [c for _, c in sel if c is not None]
        return (sum(ws) / len(ws) if ws else None, sum(cs) / len(cs) if cs else None, len(sel))

    def stop(self):
        self._stop = True


def power_context(step, seconds=2.0):
    """Context only, never the target: mean socket power and shader clock (amdsmi, 50 ms samples of firmware averages)
    while the same step repeats for `seconds`, after everything that is timed.  Next to the board's power cap it says
    whether the step runs into the cap, i.e. whether its time is set by the energy it takes rather than by idle pipes."""
    import torch

    sampler = _PowerSampler()
    time.sleep(0.2)
    t0 = time.time()
    n = 0
    while time.time() - t0 < seconds:
        step()
        torch.cuda.synchronize()
        n += 1
    t1 = time.time()
    sampler.stop()
    watts, mhz, ns = sampler.window(t0, t1)
    if sampler.error or watts is None:
        return {"error": sampler.error or "no power readings"}
    return {"mean_socket_watts": watts, "cap_watts": getattr(sampler, "cap_watts", None), "mean_shader_mhz": mhz, "samples": ns,
            "seconds": t1 - t0, "ms_per_step_meanwhile": (t1 - t0) / n * 1e3, "joules_per_step": watts * (t1 - t0) / n}


def run_mfma_ceiling(args):
    """What plain bf16 GEMMs of this path's shapes sustain on THIS box: the library's 16x16x32 mainloop (`lce_gemm_nt`,
    fp32 C; `lce_gemm_tn` for the K-major d_weight layout) next to torch.matmul (hipBLASLt, bf16 C), on all-zero operands
    and on the benchmark's distributions (N(0,1) x N(0,0.02)), with socket power and shader clock sampled meanwhile.
    The fused kernels cannot beat what the matrix pipes sustain on such data; this is the yardstick for them."""
    import torch

    from verl_amd import _abi

    lib = _abi.load()
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    sampler = _PowerSampler()
    time.sleep(0.3)
    T, H, V, vc = 16384, 3584, 152064, 8192
    shapes = [
        # name, M, N, K  (C[M, N] = A[M, K] . B[N, K]^T)
        ("forward-like 16384 x 16384 x 3584", 16384, 16384, 3584),
        ("d_logits tiles of one 8192-column chunk", T, vc, H),
        ("d_hidden GEMM of one chunk", T, H, vc),
        ("d_weight GEMM of one chunk", vc, H, T),
    ]
    g = torch.Generator(device=dev).manual_seed(99)
    cases = []
    seconds = 1.5

    def timed(fn, flops):
        fn(); fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); fn(); e1.record()
        torch.cuda.synchronize()
        reps = max(5, int(seconds * 1e3 / max(e0.elapsed_time(e1), 1e-3)))
        t0 = time.time()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.time()
        ms = e0.elapsed_time(e1) / reps
        watts, mhz, n = sampler.window(t0, t1)
        time.sleep(0.3)  # let the board cool between cases
        return {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "socket_watts": watts, "shader_mhz": mhz, "samples": n, "reps": reps}

    for data in ("zeros", "randn x 0.02 randn"):
        for name, M, N, K in shapes:
            if data == "zeros":
                A = torch.zeros(M, K, device=dev, dtype=torch.bfloat16)
                B = torch.zeros(N, K, device=dev, dtype=torch.bfloat16)
            else:
                A = torch.randn(M, K, device=dev, generator=g).bfloat16()
                B = (torch.randn(N, K, device=dev, generator=g) * 0.02).bfloat16()
            flops = 2.0 * M * N * K
            Cf = torch.empty(M, N, device=dev, dtype=torch.float32)
            r = timed(lambda: _abi.check(lib.lce_gemm_nt(A.data_ptr(), K, B.data_ptr(), K, Cf.data_ptr(), N, M, N, K, 0, 3, st), "lce_gemm_nt"), flops)
            cases.append({"shape": name, "M": M, "N": N, "K": K, "data": data, "engine": "lce_gemm_nt (16x16x32 loop, fp32 C)", **r})
            del Cf
            Cb = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            Bt = B.t()
            r = timed(lambda: torch.matmul(A, Bt, out=Cb), flops)
            cases.append({"shape": name, "M": M, "N": N, "K": K, "data": data, "engine": "torch.matmul (hipBLASLt, bf16 C)", **r})
            del Cb
            if name.startswith("d_weight"):
                # the layout the backward really uses: both operands K-major, A[K, M], B[K, N] (row strides in whole 256-column tiles)
                At, Bk = A.t().contiguous(), B.t().contiguous()
                Cf = torch.empty(M, N, device=dev, dtype=torch.float32)
                r = timed(lambda: _abi.check(lib.lce_gemm_tn(At.data_ptr(), M, Bk.data_ptr(), N, Cf.data_ptr(), N, M, N, K, 3, st), "lce_gemm_tn"), flops)
                cases.append({"shape": name, "M": M, "N": N, "K": K, "data": data, "engine": "lce_gemm_tn (16x16x32 loop, K-major operands, fp32 C)", **r})
                del At, Bk, Cf
            del A, B
    # what the memory system of this box sustains with vendor kernels, for the HBM-bound rows (few tokens, logits twins):
    # write-only (fill), read-only (sum) and read + write (copy) over 2 GiB buffers
    buf = torch.empty(1 << 29, device=dev, dtype=torch.float32)
    dst = torch.empty_like(buf)
    nbytes = buf.numel() * 4.0
    hbm = []
    for name, fn, moved in (("fill (write only)", lambda: buf.fill_(1.0), nbytes), ("sum (read only)", lambda: buf.sum(), nbytes),
                            ("copy (read + write)", lambda: dst.copy_(buf), 2.0 * nbytes)):
        r = timed(fn, 0.0)
        hbm.append({"op": f"torch {name}, 2 GiB", "ms": r["ms"], "TBps": moved / (r["ms"] * 1e-3) / 1e12, "socket_watts": r["socket_watts"],
                    "shader_mhz": r["shader_mhz"]})
    del buf, dst
    sampler.stop()
    rand = [c for c in cases if c["data"] != "zeros"]
    best_lib = max(c["tflops"] for c in rand if c["engine"].startswith("lce_"))
    best_blas = max(c["tflops"] for c in rand if c["engine"].startswith("torch"))
    # time of one fwd+bwd step of the headline workload if its four GEMM-shaped passes (8*T*V*H executed FLOP) ran at these rates
    step_flops = 8.0 * T * V * H
    out = {
        "metric": "plain bf16 GEMM rate on this box (yardstick for the fused kernels), random operands",
        "value": max(best_lib, best_blas), "unit": "TFLOP/s", "n_gpus": 1, "steps": None, "warmup": None, "ms_per_step": None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": CEILING_WORKLOAD, "seconds_per_case": seconds},
        "best_library_mainloop_tflops": best_lib, "best_hipblaslt_tflops": best_blas,
        "headline_step_ms_at_best_rate": step_flops / (max(best_lib, best_blas) * 1e12) * 1e3,
        "power_cap_watts": getattr(sampler, "cap_watts", None), "power_sampler_error": sampler.error,
        "cases": cases,
        "hbm": hbm,
        "roofline": None, "cpu_baseline": None,
    }
    print(json.dumps(out), flush=True)


SWEEP_WORKLOAD = "token-sweep"


def run_token_sweep(args):
    """Forward and forward + backward of the Qwen2.5-7B head (H=3584, V=152064, bf16) at token counts from 128 to 2048 in
    steps of 64 plus ragged counts: the band where the launchers switch code paths (at 64, 128, 512 and 1280 tokens; beyond half the hidden size the backward recomputes its logits) and
    where the bound changes from HBM (one stream of W per pass: 4 passes of [V, H] forward + backward) to the matrix
    pipes (ridge at 2.5e15 / 8e12 = 312 tokens forward, 417 forward + backward).  Each point: median of `--steps`
    runs; `frac` is the larger of the two floors (algorithmic bytes / 8 TB/s, algorithmic FLOP / 2.5 PFLOP/s) over the
    measured time.  Token tiles are 256 wide, so the matrix-pipe work is that of T rounded up to 256."""
    import torch

    from verl_amd import linear_cross_entropy

    dev = torch.device("cuda:0")
    H, V = 3584, 152064
    g = torch.Generator(device=dev).manual_seed(1234)
    w = (torch.randn(V, H, device=dev, generator=g) * 0.02).bfloat16()
    counts = sorted(set(list(range(128, 2049, 64)) + [200, 333, 500, 777, 1000, 1300, 1500, 1999]))
    n = max(3, args.steps)

    def timed(step):
        for _ in range(max(1, args.warmup)):
            step()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        ev[0].record()
        for i in range(n):
            step()
            ev[i + 1].record()
        torch.cuda.synchronize()
        return sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(n))[n // 2]

    rows = []
    for T in counts:
        h = torch.randn(T, H, device=dev, generator=g).bfloat16()
        y = torch.randint(0, V, (T,), device=dev, generator=g)
        g_lp, g_ent = torch.randn(T, device=dev, generator=g), torch.randn(T, device=dev, generator=g)

        def fwd():
            with torch.no_grad():
                linear_cross_entropy(h, w, y, 1.0, "none")

        hg, wg = h.clone().requires_grad_(True), w.requires_grad_(True)

        def fwd_bwd():
            hg.grad = None
            wg.grad = None
            lp, ent = linear_cross_entropy(hg, wg, y, 1.0, "none")
            torch.autograd.backward([lp, ent], [g_lp, g_ent])

        rec = {"T": T}
        # (streaming passes over [V, H]: up to half the hidden size in tokens the backward takes the logits the forward kept instead of a pass over W)
        for name, fn, passes, flops in (("fwd", fwd, 1.0, 2.0 * T * V * H), ("fwd_bwd", fwd_bwd, 3.0 if T <= H // 2 else 4.0, 6.0 * T * V * H)):
            ms = timed(fn)
            hbm_ms = passes * V * H * 2.0 / PEAK_HBM * 1e3
            mfma_ms = flops / PEAK_BF16 * 1e3
            rec[name] = {"ms": ms, "bound": "hbm" if hbm_ms >= mfma_ms else "mfma", "floor_ms": max(hbm_ms, mfma_ms),
                         "frac": max(hbm_ms, mfma_ms) / ms, "tokens_per_s": T / (ms * 1e-3)}
        w.requires_grad_(False)
        rows.append(rec)
    out = {
        "metric": "fraction of the applicable roofline over token counts 128..2048 (forward; forward + backward)",
        "value": min(r["fwd_bwd"]["frac"] for r in rows), "unit": "fraction (worst point, fwd+bwd)", "n_gpus": 1, "steps": n,
        "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "config": {"workload": SWEEP_WORKLOAD, "H": H, "V": V},
        "rows": rows, "roofline": None, "cpu_baseline": None,
    }
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="qwen2.5-7b-head-T16384", choices=sorted(WORKLOADS) + sorted(LOGITS_WORKLOADS) + [CEILING_WORKLOAD, SWEEP_WORKLOAD])
    ap.add_argument("--tokens", type=int, default=0, help="another token count T for the chosen head workload (its name gets the suffix @T<count>)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--variant", type=int, default=-1)
    ap.add_argument("--vchunk", type=int, default=-1)
    ap.add_argument("--split-backward", action="store_true", help="diagnostic: time the backward's three phases as separate launches")
    ap.add_argument("--dlogits-tokens-first", action="store_true", help="diagnostic: tile order of the d_logits pass")
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE", help="diagnostic: lce_set_option(KEY, VALUE)")
    ap.add_argument("--no-unfused-context", action="store_true",
                    help="skip the context figure: the reference test's unfused torch path (fp32 [T, V] logits, autograd) timed on the same GPU")
    ap.add_argument("--no-power-context", action="store_true", help="skip the two seconds of the same step under the power sampler")
    ap.add_argument("--frozen-head", action="store_true",
                    help="the weight takes no gradient (LoRA that leaves lm_head alone): the backward leaves the d_weight GEMM out")
    ap.add_argument("--print-state", action="store_true", help="print the library state that keys profiles/traffic.json and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload in LOGITS_WORKLOADS:
        run_logits_workload(args, args.workload)
        return
    if args.workload == CEILING_WORKLOAD:
        run_mfma_ceiling(args)
        return
    if args.workload == SWEEP_WORKLOAD:
        run_token_sweep(args)
        return

    import torch

    from verl_amd import _abi, linear_cross_entropy
    from verl_amd.utils.kernel import kernels as K

    lib = _abi.load()
    if args.variant >= 0:
        _abi.check(lib.lce_set_variant(args.variant), "lce_set_variant")
    if args.split_backward:
        _abi.check(lib.lce_set_option(1, 1), "lce_set_option")
    if args.dlogits_tokens_first:
        _abi.check(lib.lce_set_option(2, 1), "lce_set_option")
    for kv in args.option:
        k, v = kv.split("=")
        _abi.check(lib.lce_set_option(int(k), int(v)), "lce_set_option")
    if args.vchunk >= 0:
        K.set_vocab_chunk(args.vchunk)
    dev = torch.device("cuda:0")
    T, H, V, tau, wstd, nseq, shortest, ppo = WORKLOADS[args.workload][:8]
    workload_name = args.workload
    if args.tokens > 0:
        if nseq:
            raise SystemExit("--tokens: only for workloads without sequence structure")
        T = args.tokens
        workload_name = f"{args.workload}@T{T}"
    flags = {"variant": args.variant, "vchunk": args.vchunk, "split_backward": bool(args.split_backward),
             "options": sorted(args.option + (["2=1"] if args.dlogits_tokens_first else []))}
    if args.frozen_head:
        flags["frozen_head"] = True
    state = library_state(lib, T, H, V, flags)
    if args.print_state:
        print(json.dumps({"workload": workload_name, "state": state}), flush=True)
        return
    fwd_only = len(WORKLOADS[args.workload]) > 8 and WORKLOADS[args.workload][8]
    g = torch.Generator(device=dev).manual_seed(1234 + 2)
    h = torch.randn(T, H, device=dev, generator=g).bfloat16().requires_grad_(True)
    w = (torch.randn(V, H, device=dev, generator=g) * wstd).bfloat16().requires_grad_(not args.frozen_head)
    y = torch.randint(0, V, (T,), device=dev, generator=g)
    g_lp = torch.randn(T, device=dev, generator=g)
    g_ent = torch.randn(T, device=dev, generator=g)
    mask = torch.ones(T, device=dev)
    if nseq:
        row = T // nseq
        valid = torch.randint(shortest, row + 1, (nseq,), device=dev, generator=g)
        mask = (torch.arange(row, device=dev)[None, :] < valid[:, None]).float().reshape(T)
        g_lp, g_ent = g_lp * mask, g_ent * mask
    t_active = int(mask.sum().item())
    if ppo:
        from verl_amd.workers.utils.losses import fused_ppo_loss

        with torch.no_grad():
            lp0, _ = linear_cross_entropy(h, w, y, tau, "none")
        old_lp = lp0 + 0.05 * torch.randn(T, device=dev, generator=g)
        adv = torch.randn(nseq, device=dev, generator=g).repeat_interleave(T // nseq)
        del lp0

    if args.copy_calibration:
        src = torch.empty(1 << 30, device=dev, dtype=torch.uint8).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 1 GiB, writes 1 GiB per launch
        torch.cuda.synchronize()
        del src, dst

    def step():
        h.grad = None
        w.grad = None
        if fwd_only:
            with torch.no_grad():
                linear_cross_entropy(h, w, y, tau, "none")
            return
        lp, ent = linear_cross_entropy(h, w, y, tau, "none")
        if ppo:
            loss, _ = fused_ppo_loss(lp, ent, old_lp, adv, mask, clip_ratio=0.2, clip_ratio_c=3.0, entropy_coeff=1e-3)
            loss.backward()
        else:
            torch.autograd.backward([lp, ent], [g_lp, g_ent])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()  # (torch's current stream is the stream the library launches on)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = T / (elapsed / args.steps)
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    step_ms = {"median": per_step[len(per_step) // 2], "min": per_step[0], "max": per_step[-1]}

    # Peak device memory of one forward and one backward beyond what is live before each (outputs, saved
    # statistics, returned gradients and the workspace included), next to the bound the workspace is sized
    # under and to what ONE materialised [T, V] tensor in the input dtype would take.
    memory = None
    if not fwd_only and not ppo:
        h.grad = None
        w.grad = None
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated(dev)
        torch.cuda.reset_peak_memory_stats(dev)
        lp, ent = linear_cross_entropy(h, w, y, tau, "none")
        torch.cuda.synchronize()
        fwd_peak = torch.cuda.max_memory_allocated(dev) - base
        base = torch.cuda.memory_allocated(dev)
        torch.cuda.reset_peak_memory_stats(dev)
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
        torch.cuda.synchronize()
        bwd_peak = torch.cuda.max_memory_allocated(dev) - base
        del lp, ent
        memory = {"forward_peak_extra_bytes": fwd_peak, "backward_peak_extra_bytes": bwd_peak,
                  "returned_gradients_bytes": (T * H + V * H) * 2,
                  "workspace_bound_bytes": 0.25 * T * V * 2 + 4.0 * V * H,
                  "one_materialised_TV_tensor_bytes": T * V * 2}

    # per-kernel durations with HIP events on the launch stream (second pass, same process)
    lib.lce_profile_enable(1)
    _abi.profile_read(reset=True)
    nprof = max(2, min(args.steps, 5))
    for _ in range(nprof):
        step()
    torch.cuda.synchronize()
    prof = _abi.profile_read(reset=True)
    lib.lce_profile_enable(0)
    kernels = {k: {"ms_per_step": ms / nprof, "launches_per_step": n / nprof, "avg_ms": ms / n} for k, (ms, n) in prof.items()}
    # With few tokens (up to half the hidden size) the autograd node keeps its fp32 logits for the backward (a bounded exception to "nothing of size
    # T x V is kept"): how large that is, and the same step with the exception switched off (every backward recomputing
    # its logits, as at every larger size), timed the same way after everything else.
    logits_kept = None
    cache_bytes = 0 if fwd_only else int(lib.lce_logits_cache_bytes(T, H, V, 0))
    if cache_bytes:
        K.set_keep_logits_tokens(0)
        try:
            for _ in range(max(2, args.warmup)):
                step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(args.steps):
                step()
            torch.cuda.synchronize()
            logits_kept = {"cache_bytes": cache_bytes, "ms_per_step_when_recomputing": (time.perf_counter() - t1) / args.steps * 1e3}
        finally:
            K.set_keep_logits_tokens(None)
    # Context only, never the target: the unfused torch path of the reference's own test (materialised fp32 [T, V] logits,
    # softmax, logsumexp, cross_entropy, autograd; tests/utils/test_linear_cross_entropy.py:49-62,290-349 prints the same
    # pair of figures) on the same GPU and inputs, after everything that is timed: one warm-up, then one timed forward + backward.
    unfused = None
    if not args.no_unfused_context and not fwd_only and not ppo and not args.frozen_head and T * V <= 16384 * 152064:
        unfused = unfused_context(h, w, y, tau, g_lp, g_ent)

    # socket power against the board's cap while the step repeats (steps long enough for 50 ms samples to mean something)
    power = None
    if not args.no_power_context and ms_per_step >= 5.0:
        power = power_context(step)

    # the dominant kernel (largest share of the step) and its algorithmic FLOPs per launch:
    # algorithmic FLOPs per step of each MFMA kernel class (the recompute of the logits in the
    # backward is executed but not counted): forward 2*T*V*H; backward d_hidden + d_weight 4*Ta*V*H,
    # Ta = tokens with a non-zero upstream gradient (the others add exactly zero and are skipped)
    # (--frozen-head: one gradient GEMM instead of two)
    n_grads = 1.0 if args.frozen_head else 2.0
    algo = {"lce_fwd_kernel": 2.0 * T, "lce_bwd_chunk_kernel": 2.0 * n_grads * t_active}
    if args.split_backward:
        algo.update({"gemm_nt_kernel(d_hidden)": 2.0 * t_active, "gemm_nt_kernel(d_weight)": 2.0 * t_active})
    executed = {"lce_fwd_kernel": 2.0 * T, "lce_bwd_chunk_kernel": (2.0 + 2.0 * n_grads) * t_active, "gemm_nt_kernel(d_hidden)": 2.0 * t_active,
                "gemm_nt_kernel(d_weight)": 2.0 * t_active, "lce_bwd_ds_kernel": 2.0 * t_active}
    if cache_bytes:  # (the d_logits come from the kept logits: an elementwise kernel under the d_logits tiles' name, no recompute)
        executed["lce_bwd_chunk_kernel"] = 2.0 * n_grads * t_active
        del executed["lce_bwd_ds_kernel"]
    mfma = {k: v for k, v in kernels.items() if k in algo}
    dom = max(mfma, key=lambda k: mfma[k]["ms_per_step"])
    flops_per_launch = algo[dom] * V * H / mfma[dom]["launches_per_step"]
    achieved = flops_per_launch / (mfma[dom]["avg_ms"] * 1e-3)
    for k, v in kernels.items():
        if k in executed:
            v["executed_tflops"] = executed[k] * V * H / (v["ms_per_step"] * 1e-3) / 1e12
    if fwd_only:
        k = kernels["lce_fwd_kernel"]
        nbytes = (V * H + T * H) * 2.0
        flops = 2.0 * T * V * H
        if flops / nbytes > PEAK_BF16 / PEAK_HBM:
            # enough tokens per weight row: the matrix pipe bounds it
            out = {
                "metric": "tokens/s, forward (log-prob + entropy); % of bf16 MFMA peak",
                "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                "ms_per_step": ms_per_step, "step_ms": step_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                "dtype": "bf16", "data": "synthetic",
                "config": {"workload": workload_name, "T": T, "H": H, "V": V, "temperature": tau, "pass": "fwd"},
                "algorithmic_tflops": flops / (elapsed / args.steps) / 1e12,
                "frac_of_bf16_peak": flops / (elapsed / args.steps) / PEAK_BF16,
                "roofline": {"bound": "mfma", "kernel": "lce_fwd_kernel", "achieved": flops / (k["avg_ms"] * 1e-3) / 1e12,
                             "peak": PEAK_BF16 / 1e12, "unit": "TFLOP/s", "frac": flops / (k["avg_ms"] * 1e-3) / PEAK_BF16,
                             "traffic": measured_traffic(workload_name, "lce_fwd_kernel", state),
                             "avg_launch_ms": k["avg_ms"], "flops_per_launch": flops},
                "kernels": kernels,
                "socket_power": power,
                "cpu_baseline": None,
            }
            print(json.dumps(out), flush=True)
            return
        # one pass over W: the HBM roofline bounds it
        out = {
            "metric": "tokens/s, forward (log-prob + entropy) with few tokens; % of HBM peak",
            "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
            "data": "synthetic",
            "config": {"workload": workload_name, "T": T, "H": H, "V": V, "temperature": tau, "pass": "fwd"},
            "roofline": {"bound": "hbm", "kernel": "lce_fwd_kernel", "achieved": nbytes / (k["avg_ms"] * 1e-3) / 1e9,
                         "peak": PEAK_HBM / 1e9, "unit": "GB/s", "frac": nbytes / (k["avg_ms"] * 1e-3) / PEAK_HBM,
                         "traffic": measured_traffic(workload_name, "lce_fwd_kernel", state),
                         "avg_launch_ms": k["avg_ms"], "bytes_per_launch": nbytes},
            "kernels": kernels,
            "cpu_baseline": None,
        }
        print(json.dumps(out), flush=True)
        return
    roofline = {
        "bound": "mfma",
        "kernel": dom,
        "achieved": achieved / 1e12,
        "peak": PEAK_BF16 / 1e12,
        "unit": "TFLOP/s",
        "frac": achieved / PEAK_BF16,
        "traffic": measured_traffic(workload_name, dom, state),
        "avg_launch_ms": mfma[dom]["avg_ms"],
        "flops_per_launch": flops_per_launch,
    }
    # Algorithmic FLOPs of the step: forward 2*T*V*H, backward 4*Ta*V*H over the Ta tokens that carry an upstream gradient
    # (the mandated recompute of the logits is executed but not counted).  With Ta = T this is the reference's 6*T*V*H.
    algorithmic = (2.0 * T + 2.0 * n_grads * t_active) * V * H / (elapsed / args.steps)
    if 6.0 * T * V * H / (4.0 * V * H * 2.0) < PEAK_BF16 / PEAK_HBM and "lce_bwd_chunk_kernel" in kernels:
        # few tokens: HBM bounds the step.  Its streaming passes over [V, H] in the input dtype: W read by the forward and
        # by the d_hidden product, d_weight written; with few tokens the forward keeps the fp32 logits (T*V*4 bytes
        # written, then read by the backward) and no pass recomputes them; beyond that the d_logits tiles read W once more.
        k = kernels["lce_bwd_chunk_kernel"]
        kept = cache_bytes > 0
        passes_bwd = n_grads if kept else 1.0 + n_grads
        nbytes = passes_bwd * V * H * 2.0 / k["launches_per_step"]  # (W read for d_hidden, d_weight written; --frozen-head: W read)
        step_bytes = (1.0 + passes_bwd) * V * H * 2.0 + (2.0 * T * V * 4.0 if kept else 0.0)
        roofline = {"bound": "hbm", "kernel": "lce_bwd_chunk_kernel", "achieved": nbytes / (k["avg_ms"] * 1e-3) / 1e9,
                    "peak": PEAK_HBM / 1e9, "unit": "GB/s", "frac": nbytes / (k["avg_ms"] * 1e-3) / PEAK_HBM,
                    "traffic": measured_traffic(workload_name, "lce_bwd_chunk_kernel", state),
                    "avg_launch_ms": k["avg_ms"], "bytes_per_launch": nbytes, "logits_kept": kept,
                    "step_bytes": step_bytes, "step_GBps": step_bytes / (elapsed / args.steps) / 1e9}
    out = {
        "metric": "fwd+bwd tokens/s, 7B lm-head logprob+entropy; % of bf16 MFMA peak",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "step_ms": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": workload_name, "T": T, "H": H, "V": V, "temperature": tau,
                   "pass": ("fwd+ppo_loss+bwd" if ppo else "fwd+bwd") + (" (d_hidden only: frozen head)" if args.frozen_head else ""),
                   "tokens_with_gradient": t_active},
        "memory": memory,
        "logits_kept": logits_kept,
        "algorithmic_tflops": algorithmic / 1e12,
        "frac_of_bf16_peak": algorithmic / PEAK_BF16,
        # tokens without upstream gradient are skipped by the backward: `value` counts them (they are part of the batch),
        # the FLOP figures above do not; 6*T*V*H per step over every token is given separately and is NOT a fraction of peak
        "row_skip": t_active < T,
        "per_token_accounting_tflops": 6.0 * T * V * H / (elapsed / args.steps) / 1e12,
        # what the kernels execute: forward on T tokens, recompute + two GEMMs on the tokens with gradient
        "executed_tflops": (2.0 * T + (2.0 + 2.0 * n_grads) * t_active) * V * H / (elapsed / args.steps) / 1e12,
        "roofline": roofline,
        "kernels": kernels,
        "unfused_torch_same_gpu": unfused,
        "socket_power": power,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(),
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
