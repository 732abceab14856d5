"""AWQ linear method on MI355X.

Mirrors ``AWQGCUConfig`` / ``AWQGCULinearMethod``
(vllm_gcu/kernels/quantization/awq.py:21-134).  The reference repacks on the CPU
with ``zeros_in_int8=True``; here the checkpoint tensors go through the device
repack kernels (AWQ interleave undone, zero-points packed as int4).
"""
from typing import Optional

import torch
from torch.nn import Parameter

from .. import _custom_ops as ops
from . import rearrange
from .utils import register_gcu_quantization_config


@register_gcu_quantization_config("awq_gcu")
class AWQGCUConfig:
    def __init__(self, weight_bits: int, group_size: int, zero_point: bool = True):
        if weight_bits != 4:
            raise ValueError(f"AWQ supports 4-bit weights only, got {weight_bits}")
        self.weight_bits = weight_bits
        self.group_size = group_size
        self.zero_point = zero_point
        self.pack_factor = 32 // weight_bits

    @classmethod
    def get_name(cls) -> str:
        return "awq_gcu"

    def get_supported_act_dtypes(self):
        return [torch.half, torch.bfloat16]

    @classmethod
    def from_config(cls, config):
        return cls(config.get("w_bit", config.get("bits", 4)), config.get("q_group_size", config.get("group_size", 128)),
                   config.get("zero_point", True))

    def get_quant_method(self, layer=None, prefix: str = ""):
        return AWQGCULinearMethod(self)


class AWQGCULinearMethod:
    def __init__(self, quant_config: AWQGCUConfig):
        self.quant_config = quant_config

    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size,
                       output_size, params_dtype, **extra_weight_attrs):
        cfg = self.quant_config
        out = sum(output_partition_sizes)
        groups = input_size_per_partition // cfg.group_size
        layer.register_parameter("qweight", Parameter(torch.empty(
            input_size_per_partition, out // cfg.pack_factor, dtype=torch.int32), requires_grad=False))
        layer.register_parameter("qzeros", Parameter(torch.empty(
            groups, out // cfg.pack_factor, dtype=torch.int32), requires_grad=False))
        layer.register_parameter("scales", Parameter(torch.empty(groups, out, dtype=params_dtype),
                                                     requires_grad=False))

    def process_weights_after_loading(self, layer) -> None:
        qweight, qzeros = rearrange.rearrange_uint4_int32_awq(layer.qweight.data, layer.qzeros.data)
        layer.qweight = Parameter(qweight, requires_grad=False)
        layer.qzeros = Parameter(qzeros, requires_grad=False)

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        if x.numel() == 0:
            return torch.empty([0, layer.qweight.shape[-1]], dtype=x.dtype, device=x.device)
        out_shape = x.shape[:-1] + (layer.qweight.shape[-1],)
        # positional order of the operator: (x, kernel, scales, zeros, split_k_iters, ...) (awq.py:125-133)
        out = ops.awq_gemm_gcu(x.reshape(-1, x.shape[-1]), layer.qweight, layer.scales, layer.qzeros,
                               self.quant_config.pack_factor, bias=bias, group_size=self.quant_config.group_size)
        return out.reshape(out_shape)
