"""MI355X-native fused lm-head log-prob + entropy (drop-in for verl's ``linear_cross_entropy`` path).

Public surface mirrors the reference's module layout:

* ``verl_amd.utils.kernel.linear_cross_entropy.linear_cross_entropy``
* ``verl_amd.utils.kernel.kernels`` (host launchers, enums, ``set_backward_method``)
* ``verl_amd.utils.torch_functional`` (``logprobs_from_logits``, ``entropy_from_logits``, masked reductions)
* ``verl_amd.utils.experimental.torch_functional.FusedLinearForPPO``

All device work goes through the C ABI of ``verl_amd/lib/liblce_gfx950.so`` (see ``include/lce_abi.h``);
there is no CPU or eager fallback: calling an op without the built library raises.
"""

__version__ = "0.1.0"

from .utils.kernel.linear_cross_entropy import LinearCrossEntropy, linear_cross_entropy  # noqa: E402,F401
