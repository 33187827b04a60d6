"""Selects the fused-kernel forward for a HF causal LM.

Same entry point as the reference's ``patch_forward_with_backends``
(``verl/models/transformers/monkey_patch.py:234-291``).  Every backend name verl's configuration can carry keeps
working, with the output shape that backend has in the reference: ``triton`` (and the explicit ``hip``) install the
forward that returns ``linear_cross_entropy``'s flat fp32 vectors, ``torch`` (verl's default ``impl_backend``) and
``liger`` the one that goes through ``FusedLinearForPPO`` and returns ``[batch, seq]`` outputs with the entropy in the
hidden dtype; all of them run the same HIP kernels.  The model types the reference gives forwards of their own
(``:255-274``: qwen2_vl / qwen2_5_vl, qwen3_vl / qwen3_vl_moe, glm4v, qwen3_5 / qwen3_5_moe) get theirs from
``vlm_common``; every other model type gets the dense pair (``:275-279``).
"""

from __future__ import annotations

_FLAT_BACKENDS = ("hip", "triton")
_SHAPED_BACKENDS = ("torch", "liger")


def patch_forward_with_backends(model, use_fused_kernels: bool = False, fused_kernels_backend: str = None):
    if not use_fused_kernels or fused_kernels_backend not in _FLAT_BACKENDS + _SHAPED_BACKENDS:
        print(
            f"Skipping monkey patch for {model.__class__.__name__} as use_fused_kernels is "
            f"{use_fused_kernels} or fused_kernels_backend is {fused_kernels_backend}"
        )
        return
    from . import vlm_common

    model_type = getattr(model.config, "model_type", None)
    if model_type in vlm_common.MROPE_TYPES + vlm_common.PLAIN_TYPES:
        forward_with_hip_backend, forward_with_torch_backend = vlm_common.make_forwards(model_type)
    else:
        from .dense_common import forward_with_hip_backend, forward_with_torch_backend

    model._verl_fused_kernels_backend = fused_kernels_backend
    flat = fused_kernels_backend in _FLAT_BACKENDS
    model.__class__.forward = forward_with_hip_backend if flat else forward_with_torch_backend
    print(f"Using HIP kernels behind the {fused_kernels_backend} backend for fused kernels in {model.__class__.__name__}")
