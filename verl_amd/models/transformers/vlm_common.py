"""Fused-head forwards for the multimodal model types, twins of the reference's per-model pairs
``forward_with_torch_backend`` / ``forward_with_triton_backend`` in ``verl/models/transformers/qwen2_vl.py:490-566``
(also used for ``qwen2_5_vl``), ``qwen3_vl.py:344-422`` (also ``qwen3_vl_moe``), ``glm4v.py:469-545`` and
``qwen3_5.py:556-660`` (also ``qwen3_5_moe``).

Those pairs differ from the dense ones only in how the final hidden states are produced; the head (next-token targets,
``linear_cross_entropy`` or ``FusedLinearForPPO``, the output fields) is the same in all of them, so here ONE pair of
forwards takes the way to the hidden states as a parameter:

* ``mrope`` (qwen2_vl, qwen2_5_vl, glm4v): ``self.model(...)`` with the image / video inputs named and ``position_ids``
  required in the layout the reference's data pipeline produces, ``(4, batch, seq)`` (text positions stacked on the
  three vision axes; ``qwen2_vl.py:402-413``, ``glm4v.py:394-401``);
* ``plain`` (qwen3_vl, qwen3_vl_moe, qwen3_5, qwen3_5_moe): ``self.model(input_ids, **kwargs)``
  (``qwen3_vl.py:397``, ``qwen3_5.py:625-629``; ``cu_seqlens`` / ``cu_seqlens_cpu`` travel on when given).

What is NOT here: the reference's attention and input-embedding patches for these models (their sequence-parallel and
old-transformers paths); with ``transformers >= 4.54`` the unpatched ``self.model`` is what the reference itself
calls.  Under sequence parallelism the caller passes ``shift_labels`` (rolled on the global sequence), as the
reference's engines do; the local roll below is only right for whole sequences.
"""

from __future__ import annotations

import functools
import sys
from dataclasses import dataclass
from typing import Optional

import torch

from .dense_common import CausalLMOutputForPPO, _flat_head, _shaped_head

MROPE_TYPES = ("qwen2_vl", "qwen2_5_vl", "glm4v")
PLAIN_TYPES = ("qwen3_vl", "qwen3_vl_moe", "qwen3_5", "qwen3_5_moe")


def process_position_ids(position_ids: torch.Tensor) -> torch.Tensor:
    """The reference's check (``qwen2_vl.py:402-413``): text positions stacked on the three vision axes."""
    if position_ids is None or position_ids.ndim != 3 or position_ids.size(0) != 4:
        raise ValueError("position_ids should be a 3D tensor of shape (4, batch_size, seq_length).")
    return position_ids


def _hidden_mrope(model, input_ids, attention_mask=None, position_ids=None, pixel_values=None, pixel_values_videos=None,
                  image_grid_thw=None, video_grid_thw=None, **kwargs):
    return model.model(input_ids=input_ids, attention_mask=attention_mask, position_ids=process_position_ids(position_ids),
                       pixel_values=pixel_values, pixel_values_videos=pixel_values_videos, image_grid_thw=image_grid_thw,
                       video_grid_thw=video_grid_thw, **kwargs)


def _hidden_plain(model, input_ids, cu_seqlens=None, cu_seqlens_cpu=None, **kwargs):
    if cu_seqlens is not None:
        kwargs["cu_seqlens"] = cu_seqlens
    if cu_seqlens_cpu is not None:
        kwargs["cu_seqlens_cpu"] = cu_seqlens_cpu
    return model.model(input_ids, **kwargs)


@functools.lru_cache(maxsize=None)
def _output_class(model_cls):
    """The model's own ``...CausalLMOutputWithPast`` plus ``log_probs`` and ``entropy`` (what the reference declares per
    model, e.g. ``Qwen2VLCausalLMOutputForPPO``, ``qwen2_vl.py:416-419``); the dense output type where the model's module
    has no such class."""
    module = sys.modules.get(model_cls.__module__)
    bases = [v for k, v in vars(module).items() if k.endswith("CausalLMOutputWithPast") and isinstance(v, type)] if module else []
    if len(bases) != 1:
        return CausalLMOutputForPPO

    @dataclass
    class _Output(bases[0]):
        log_probs: Optional[torch.FloatTensor] = None
        entropy: Optional[torch.FloatTensor] = None

    _Output.__name__ = _Output.__qualname__ = bases[0].__name__.replace("WithPast", "ForPPO")
    return _Output


def _targets(name, input_ids, labels, shift_labels):
    if shift_labels is not None:
        return shift_labels
    source = labels if labels is not None else input_ids
    if source is None:
        raise RuntimeError(f"To use {name}, either labels or input_ids must be provided.")
    return torch.roll(source, shifts=-1, dims=-1)


def make_forwards(model_type: str):
    """(forward with the flat fp32 outputs of ``linear_cross_entropy``, forward with ``FusedLinearForPPO``'s shaped
    outputs) for one of the multimodal model types; both are plain functions to install as ``model.__class__.forward``."""
    if model_type in MROPE_TYPES:
        hidden_of = _hidden_mrope
    elif model_type in PLAIN_TYPES:
        hidden_of = _hidden_plain
    else:
        raise NotImplementedError(f"model_type {model_type} is not one of {MROPE_TYPES + PLAIN_TYPES}")

    def run(self, head, name, input_ids, labels, temperature, shift_labels, kwargs):
        targets = _targets(name, input_ids, labels, shift_labels)  # (fails before the model runs, not after)
        outputs = hidden_of(self, input_ids, **kwargs)
        log_probs, entropy = head(self, outputs[0], targets, temperature)
        return _output_class(type(self))(log_probs=log_probs, entropy=entropy, hidden_states=outputs.hidden_states)

    def forward_with_hip_backend(self, input_ids=None, labels=None, temperature: float = 1.0, shift_labels=None, **kwargs):
        return run(self, _flat_head, "forward_with_hip_backend", input_ids, labels, temperature, shift_labels, kwargs)

    def forward_with_torch_backend(self, input_ids=None, labels=None, temperature: float = 1.0, shift_labels=None, **kwargs):
        return run(self, _shaped_head, "forward_with_torch_backend", input_ids, labels, temperature, shift_labels, kwargs)

    return forward_with_hip_backend, forward_with_torch_backend
