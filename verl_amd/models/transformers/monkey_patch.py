"""Selects the fused-kernel forward for a HF causal LM.

Same entry point as the reference's ``patch_forward_with_backends``
(``verl/models/transformers/monkey_patch.py:234-291``).  Every backend name verl's configuration can
carry (``triton``, ``torch``, ``liger``) and the explicit ``hip`` select the one HIP path here, so an
existing ``fused_kernel_options.impl_backend`` keeps working.  Only dense text models are covered
(the reference's VLM variants differ in how they build hidden states, not in the head).
"""

from __future__ import annotations

_BACKENDS = ("hip", "triton", "torch", "liger")
_VLM_TYPES = ("qwen2_5_vl", "qwen2_vl", "qwen3_vl", "qwen3_vl_moe", "glm4v", "qwen3_5", "qwen3_5_moe")


def patch_forward_with_backends(model, use_fused_kernels: bool = False, fused_kernels_backend: str = None):
    if not use_fused_kernels or fused_kernels_backend not in _BACKENDS:
        print(
            f"Skipping monkey patch for {model.__class__.__name__} as use_fused_kernels is "
            f"{use_fused_kernels} or fused_kernels_backend is {fused_kernels_backend}"
        )
        return
    if getattr(model.config, "model_type", None) in _VLM_TYPES:
        raise NotImplementedError(f"model_type {model.config.model_type}: only dense text models are adapted")
    from .dense_common import forward_with_hip_backend

    model._verl_fused_kernels_backend = fused_kernels_backend
    model.__class__.forward = forward_with_hip_backend
    print(f"Using HIP backend for fused kernels in {model.__class__.__name__}")
