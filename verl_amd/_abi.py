"""ctypes binding of the C ABI declared in ``include/lce_abi.h``."""

from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("LCE_LIBRARY_PATH") or os.path.join(_HERE, "lib", "liblce_gfx950.so")

DTYPE_BF16, DTYPE_F32, DTYPE_F16 = 0, 1, 2
ABI_VERSION = 10

# every symbol include/lce_abi.h declares: name -> (restype, argtypes)
_c = ctypes
_p, _i64, _i, _f, _sz = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_float, _c.c_size_t
SYMBOLS = {
    "lce_abi_version": (_i, []),
    "lce_last_error": (_c.c_char_p, []),
    "lce_forward_workspace_bytes": (_sz, [_i64, _i64, _i64, _i]),
    "lce_forward": (_i, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "lce_forward_static": (_i, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p]),
    "lce_backward_workspace_bytes": (_sz, [_i64, _i64, _i64, _i, _i64]),
    "lce_backward": (
        _i,
        [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _i64, _p],
    ),
    "lce_backward_f32": (
        _i,
        [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _i64, _p],
    ),
    "lce_logits_cache_max_tokens": (_i64, [_i64, _i]),
    "lce_logits_cache_bytes": (_sz, [_i64, _i64, _i64, _i]),
    "lce_forward_keep_logits": (
        _i,
        [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p, _sz, _p, _sz, _p],
    ),
    "lce_backward_from_logits": (
        _i,
        [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p, _p, _i, _p, _sz, _i64, _p, _sz, _p],
    ),
    "lce_forward_shard": (_i, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i, _f, _p, _p, _sz, _p]),
    "lce_merge_shards": (_i, [_p, _i, _i64, _i, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "lce_backward_shard": (
        _i,
        [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i, _f, _i, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _i64, _p],
    ),
    "lce_logits_forward": (_i, [_p, _i64, _p, _i64, _i64, _i, _p, _p, _p, _p]),
    "lce_logits_backward": (_i, [_p, _i64, _p, _i64, _i64, _i, _p, _p, _p, _p, _i64, _p]),
    "lce_logits_sum_pi_squared": (_i, [_p, _i64, _i64, _i64, _i, _p, _p, _p]),
    "lce_logits_sum_pi_squared_backward": (_i, [_p, _i64, _i64, _i64, _i, _p, _p, _p, _p, _i64, _p]),
    "lce_ppo_loss_workspace_bytes": (_sz, [_i64, _i64]),
    "lce_ppo_loss": (_i, [_p, _p, _p, _p, _p, _p, _p, _i, _f, _i64, _i64, _i, _f, _f, _f, _f, _f, _f, _f, _f, _p, _p, _p, _p, _sz, _p]),
    "lce_ppo_loss_packed": (_i, [_p, _p, _i64, _p, _p, _p, _p, _p, _p, _p, _i, _f, _i64, _i64, _i, _f, _f, _f, _f, _f, _f, _f, _f, _p, _p, _p, _p, _sz, _p]),
    "lce_gemm_nt": (_i, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i, _i, _p]),
    "lce_gemm_tn": (_i, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i, _p]),
    "lce_set_variant": (_i, [_i]),
    "lce_num_variants": (_i, []),
    "lce_set_option": (_i, [_i, _i64]),
    "lce_profile_enable": (_i, [_i]),
    "lce_profile_num_classes": (_i, []),
    "lce_profile_class_name": (_c.c_char_p, [_i]),
    "lce_profile_read": (_i, [_p, _p, _i]),
}

_lib = None
_lock = threading.Lock()


class LceError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Loads the HIP library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise LceError(
                f"{LIB_PATH} is missing: build it with `python -m verl_amd.build` (needs hipcc, targets gfx950). "
                "verl_amd has no CPU or eager fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.lce_abi_version() != ABI_VERSION:
            raise LceError(f"ABI version mismatch: library {lib.lce_abi_version()}, binding {ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().lce_last_error().decode(errors="replace")
        if "Invalid reduction" in msg:
            raise ValueError(msg)
        raise LceError(f"{what} failed ({rc}): {msg}")


def dtype_code(dtype) -> int:
    import torch

    if dtype == torch.bfloat16:
        return DTYPE_BF16
    if dtype == torch.float32:
        return DTYPE_F32
    if dtype == torch.float16:
        return DTYPE_F16
    raise NotImplementedError(f"verl_amd supports bfloat16, float16 and float32 inputs, got {dtype}")


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def current_stream(device) -> int:
    import torch

    return torch.cuda.current_stream(device).cuda_stream


def profile_read(reset: bool = True) -> dict[str, tuple[float, int]]:
    """{kernel class: (total ms, launches)} since profiling was enabled / last reset."""
    lib = load()
    n = lib.lce_profile_num_classes()
    ms = (ctypes.c_double * n)()
    cnt = (ctypes.c_int64 * n)()
    check(lib.lce_profile_read(ctypes.addressof(ms), ctypes.addressof(cnt), 1 if reset else 0), "lce_profile_read")
    return {lib.lce_profile_class_name(i).decode(): (ms[i], cnt[i]) for i in range(n) if cnt[i] > 0}
