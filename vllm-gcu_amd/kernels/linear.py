"""Linear-layer forwards that pass an activation scale through to the quantised method.

Mirrors the ``forward`` of ``MergedReplicatedLinear`` and ``CustomMergedColumnParallelLinear``
(vllm_gcu/kernels/linear.py:117-129, 132-150): a caller that has already quantised the activations to
fp8 (a fused norm + quantise prologue) hands the per-token-group scales over as ``x_scale`` /
``input_scale``; only the ``fp8_gcu`` method accepts them.  The classes are mix-ins over whatever linear
base class the serving framework provides (vLLM's ``ReplicatedLinear`` / ``MergedColumnParallelLinear``):
they read ``bias``, ``skip_bias_add``, ``return_bias`` and ``quant_method`` from it.
"""
from typing import Optional

import torch


class XScaleForwardMixin:
    def forward(self, x: torch.Tensor, x_scale: Optional[torch.Tensor] = None):
        bias = self.bias if not self.skip_bias_add else None
        assert self.quant_method is not None
        if x_scale is not None:
            assert self.quant_method.quant_config.get_name() == "fp8_gcu"
            output = self.quant_method.apply(self, x, bias, x_scale)
        else:
            output = self.quant_method.apply(self, x, bias)
        output_bias = self.bias if self.skip_bias_add else None
        if not getattr(self, "return_bias", True):
            return output
        return output, output_bias


class MergedReplicatedLinearMixin(XScaleForwardMixin):
    """vllm_gcu/kernels/linear.py:20-129 keeps the merged q_a / kv_a projection of an MLA layer in one
    replicated linear; the loader side is vLLM's, the forward is the pass-through above."""


class CustomMergedColumnParallelLinearMixin(XScaleForwardMixin):
    """vllm_gcu/kernels/linear.py:132-150 (same forward, the argument is called ``input_scale`` there)."""

    def forward(self, input_, input_scale: Optional[torch.Tensor] = None):
        return XScaleForwardMixin.forward(self, input_, input_scale)
