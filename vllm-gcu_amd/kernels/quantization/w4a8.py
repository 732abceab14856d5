"""W4A8-fp8 MoE method on MI355X: symmetric int4 experts, fp8 activations with
one static scale per GEMM.

Mirrors ``W4A8Config`` / ``MoeW4A8Method`` (vllm_gcu/kernels/quantization/
w4a8.py:26-502): AWQ-packed checkpoint experts (``int32 [E, K, N/8]``, or int8
``[E, K/2, N]`` when the checkpoint is marked ``rearranged``), fp32 group scales
``[E, K/g, N]``, ``w13_input_scale`` / ``w2_input_scale`` loaded as the
reciprocal of the checkpoint value (w4a8.py:484-497) and their reciprocals
``*_input_scale_rec`` handed to the GEMM (w4a8.py:222-235).  The reference keeps
experts as int8 half-group tensors ``[E, N, K/2]`` for its vendor kernel; here
they become ``int32 [E, K/8, N]`` slab tensors (unsigned nibbles, implicit
zero-point 8).  Dense layers of such a checkpoint are block-fp8
(``Fp8GCULinearMethod``, w4a8.py:94-97).
"""
from typing import Any, Dict, List, Optional

import torch
from torch.nn import Parameter

from ..fused_moe import select_experts
from ..modular_experts import TritonExpertsPad
from ..modular_kernel import FusedMoEModularKernel
from ..prepare_finalize import MoEPrepareAndFinalizeNoEP
from . import rearrange
from .utils import register_gcu_quantization_config


@register_gcu_quantization_config("w4a8_gcu")
class W4A8Config:
    def __init__(self, linear_quant_method: str = "w4a8", weight_bits: int = 4, group_size: int = 128,
                 has_zp: bool = False, lm_head_quantized: bool = False,
                 modules_to_not_convert: Optional[List[str]] = None,
                 full_config: Optional[Dict[str, Any]] = None):
        if weight_bits != 4:
            raise ValueError("w4a8: experts are 4-bit")
        if group_size != 128:
            # the reference calls its kernel with group_k = 128 whatever the config says (fused_moe.py:192)
            raise ValueError("w4a8: expert group size is 128")
        self.linear_quant_method = linear_quant_method
        self.weight_bits = weight_bits
        self.group_size = group_size
        self.has_zp = has_zp
        self.bit8_pack_factor = 8 // weight_bits
        self.pack_factor = 32 // weight_bits
        self.lm_head_quantized = lm_head_quantized
        self.modules_to_not_convert = modules_to_not_convert or []
        self.full_config = full_config or {}
        # dense layers: block-fp8 (w4a8.py:52-56)
        self.weight_block_size = [128, 128]
        self.rearranged = bool(self.full_config.get("rearranged", False))

    @classmethod
    def get_name(cls) -> str:
        return "w4a8_gcu"

    @classmethod
    def get_supported_act_dtypes(cls):
        return [torch.bfloat16, torch.half]

    @classmethod
    def from_config(cls, config: Dict[str, Any]) -> "W4A8Config":
        return cls(config["quant_method"], config["bits"], config["group_size"], config["zero_point"],
                   config.get("lm_head", False), config.get("modules_to_not_convert"), config)

    def get_quant_method(self, layer=None, prefix: str = "", moe: bool = False):
        if any(name in prefix for name in self.modules_to_not_convert):
            return None
        if moe:
            return MoeW4A8Method(self)
        from .fp8 import Fp8GCULinearMethod
        return Fp8GCULinearMethod(self)


class MoeW4A8Method:
    def __init__(self, quant_config: W4A8Config):
        self.quant_config = quant_config
        self.fused_experts = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), self.select_gemm_impl())

    def select_gemm_impl(self, prepare_finalize=None, moe=None):
        # w4a8.py:393-402: fp8 activations, no block shape (one static scale)
        return TritonExpertsPad(use_fp8_w8a8=True, block_shape=None)

    def create_weights(self, layer, num_experts: int, hidden_size: int, intermediate_size_per_partition: int,
                       params_dtype: torch.dtype, **extra_weight_attrs) -> None:
        """Parameter shapes of w4a8.py:237-391 (v1: AWQ int32, v2: rearranged int8)."""
        cfg = self.quant_config
        g, inter = cfg.group_size, intermediate_size_per_partition

        def reg(name, t):
            layer.register_parameter(name, Parameter(t, requires_grad=False))

        if cfg.rearranged:
            reg("w13_qweight", torch.empty(num_experts, hidden_size // cfg.bit8_pack_factor, 2 * inter,
                                           dtype=torch.int8))
            reg("w2_qweight", torch.empty(num_experts, inter // cfg.bit8_pack_factor, hidden_size,
                                          dtype=torch.int8))
        else:
            reg("w13_qweight", torch.empty(num_experts, hidden_size, 2 * inter // cfg.pack_factor,
                                           dtype=torch.int32))
            reg("w2_qweight", torch.empty(num_experts, inter, hidden_size // cfg.pack_factor, dtype=torch.int32))
        reg("w13_scales", torch.zeros(num_experts, hidden_size // g, 2 * inter, dtype=torch.float32))
        reg("w2_scales", torch.zeros(num_experts, inter // g, hidden_size, dtype=torch.float32))
        reg("w13_input_scale", torch.ones(1, dtype=torch.float32))
        reg("w2_input_scale", torch.ones(1, dtype=torch.float32))

    @staticmethod
    def load_input_scale(param: torch.Tensor, loaded_weight: torch.Tensor) -> None:
        """The checkpoint's input scales are stored reciprocally (w4a8.py:484-497)."""
        assert param.size() == loaded_weight.size()
        param.data.copy_(1.0 / loaded_weight)

    def process_weights_after_loading(self, layer) -> None:
        for name in ("w13", "w2"):
            qw = getattr(layer, f"{name}_qweight").data
            if qw.dtype == torch.int32:
                # AWQ interleave, unsigned nibbles; "w - 8" of rearrange.py:104-106 is the implicit zero 8
                w, _ = rearrange.rearrange_uint4_int32_awq(qw, None)
            else:
                E, K2, N = qw.shape          # int8 [E, K/2, N], half-groups of 32 rows, signed nibbles
                w = rearrange.from_reference_w4a8(qw.contiguous().view(E, N, K2))
            setattr(layer, f"{name}_qweight", Parameter(w, requires_grad=False))
            s = getattr(layer, f"{name}_input_scale").data
            layer.register_parameter(f"{name}_input_scale_rec",
                                     Parameter((1.0 / s.to(torch.float32)), requires_grad=False))

    def apply(self, layer, x, router_logits, top_k: int, renormalize: bool, use_grouped_topk: bool = False,
              topk_group=None, num_expert_group=None, global_num_experts: int = -1, expert_map=None,
              custom_routing_function=None, scoring_func: str = "softmax", e_score_correction_bias=None,
              apply_router_weight_on_input: bool = False, activation: str = "silu"):
        topk_weights, topk_ids = select_experts(x, router_logits, top_k, use_grouped_topk, renormalize,
                                                topk_group, num_expert_group, custom_routing_function,
                                                scoring_func, e_score_correction_bias)
        return self.fused_experts(x, layer.w13_qweight, layer.w2_qweight, topk_weights=topk_weights,
                                  topk_ids=topk_ids, inplace=False, activation=activation,
                                  global_num_experts=global_num_experts, expert_map=expert_map,
                                  w1_scale=layer.w13_scales, w2_scale=layer.w2_scales,
                                  a1_scale=layer.w13_input_scale, a2_scale=layer.w2_input_scale,
                                  apply_router_weight_on_input=apply_router_weight_on_input,
                                  a1_scale_rec=layer.w13_input_scale_rec, a2_scale_rec=layer.w2_input_scale_rec)
