"""GPTQ linear method on MI355X.

Mirrors ``GPTQGCUConfig`` / ``GPTQGCULinearMethod``
(vllm_gcu/kernels/quantization/gptq.py:31-296): same parameter names and
checkpoint shapes in ``create_weights``, same ``apply`` call into
``ops.gptq_gemm_gcu``.  ``process_weights_after_loading`` differs on purpose: the
reference unpacks on the CPU into its uint8 half-group layout with float
zeros; here a device kernel converts the checkpoint tensors to the slab layout
and keeps the zero-points as packed integers.
"""
from typing import Optional

import torch
from torch.nn import Parameter

from .. import _custom_ops as ops
from . import rearrange
from .utils import register_gcu_quantization_config


@register_gcu_quantization_config("gptq_gcu")
class GPTQGCUConfig:
    def __init__(self, weight_bits: int, group_size: int, desc_act: bool = False, lm_head_quantized: bool = False):
        if weight_bits not in (4, 8):
            raise ValueError(f"GPTQ on MI355X supports 4/8-bit weights, got {weight_bits}")
        self.weight_bits = weight_bits
        self.group_size = group_size
        self.desc_act = desc_act
        self.lm_head_quantized = lm_head_quantized
        self.pack_factor = 32 // weight_bits

    @classmethod
    def get_name(cls) -> str:
        return "gptq_gcu"

    @classmethod
    def get_supported_act_dtypes(cls):
        return [torch.half, torch.bfloat16]

    @classmethod
    def from_config(cls, config):
        return cls(config["bits"], config["group_size"], config.get("desc_act", False),
                   config.get("lm_head", False))

    def get_quant_method(self, layer=None, prefix: str = ""):
        return GPTQGCULinearMethod(self)


class GPTQGCULinearMethod:
    def __init__(self, quant_config: GPTQGCUConfig):
        self.quant_config = quant_config

    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size,
                       output_size, params_dtype, **extra_weight_attrs):
        cfg = self.quant_config
        group_size = cfg.group_size if cfg.group_size != -1 else input_size
        if input_size_per_partition % group_size != 0:
            raise ValueError("The input size is not aligned with the quantized weight shape "
                             "(gptq.py:128-133).")
        out = sum(output_partition_sizes)
        groups = input_size_per_partition // group_size
        layer.register_parameter("qweight", Parameter(torch.empty(
            input_size_per_partition // cfg.pack_factor, out, dtype=torch.int32), requires_grad=False))
        layer.register_parameter("g_idx", Parameter(torch.tensor(
            [i // group_size for i in range(input_size_per_partition)], dtype=torch.int32), requires_grad=False))
        layer.register_parameter("qzeros", Parameter(torch.empty(
            groups, out // cfg.pack_factor, dtype=torch.int32), requires_grad=False))
        layer.register_parameter("scales", Parameter(torch.empty(groups, out, dtype=params_dtype),
                                                     requires_grad=False))

    def process_weights_after_loading(self, layer) -> None:
        cfg = self.quant_config
        g_idx = layer.g_idx.data
        gs = cfg.group_size if cfg.group_size != -1 else g_idx.numel()
        if cfg.weight_bits == 4:
            expect = torch.arange(g_idx.numel(), device=g_idx.device, dtype=g_idx.dtype) // gs
            if not torch.equal(g_idx, expect):
                raise ValueError("act-order (non-contiguous g_idx) checkpoints are not supported "
                                 "(gptq.py:141-143)")
            qweight, qzeros = rearrange.rearrange_uint4_int32_gptq(layer.qweight.data, layer.qzeros.data)
            layer.qweight = Parameter(qweight, requires_grad=False)
            layer.qzeros = Parameter(qzeros, requires_grad=False)
        else:
            # symmetric 8-bit only: stored zero 127 (+1 = 128) (gptq.py:262-270)
            if not torch.all(layer.qzeros.data.view(torch.int8) == 127):
                raise ValueError("only support sym quant")
            w = layer.qweight.data.T.contiguous().view(torch.uint8).to(torch.int16) - 128
            layer.qweight = Parameter(w.to(torch.int8), requires_grad=False)      # [N, K]
            layer.qzeros = None
            if cfg.group_size == -1:
                layer.scales = Parameter(layer.scales.data.squeeze(0), requires_grad=False)

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        n_out = layer.qweight.shape[-1] if self.quant_config.weight_bits == 4 else layer.qweight.shape[0]
        if x.numel() == 0:
            return torch.empty([0, n_out], dtype=x.dtype, device=x.device)
        zeros = layer.qzeros if layer.qzeros is not None else torch.empty(0, dtype=torch.int32, device=x.device)
        return ops.gptq_gemm_gcu(x, layer.qweight, zeros, layer.scales, layer.g_idx,
                                 self.quant_config.weight_bits, bias=bias,
                                 group_size=self.quant_config.group_size)
