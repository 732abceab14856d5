"""int4 weight-only MoE method on MI355X.

Mirrors ``MoeWNA16GCUMethod`` (vllm_gcu/kernels/quantization/moe_wna16.py:160-643):
per-expert GPTQ / AWQ checkpoint tensors are repacked once
(``process_weights_after_loading``), ``select_gemm_impl`` picks the fused
experts with ``use_int4_w4a16`` and ``block_shape=[0, group_size]``
(moe_wna16.py:574-584) and ``apply`` runs them.  The reference stores each
expert transposed as uint8 ``[E, N, K/2]`` with float zeros; here experts are
``int32 [E, K/8, N]`` slab tensors with packed int4 zero-points.
"""
import torch
from torch.nn import Parameter

from ..fused_moe import select_experts
from ..modular_experts import TritonExpertsPad
from ..modular_kernel import FusedMoEModularKernel
from ..prepare_finalize import MoEPrepareAndFinalizeNoEP
from . import rearrange
from .utils import register_gcu_quantization_config


@register_gcu_quantization_config("moe_wna16_gcu")
class MoeWNA16GCUConfig:
    def __init__(self, linear_quant_method: str, weight_bits: int, group_size: int, has_zp: bool):
        if weight_bits != 4:
            raise ValueError("only 4-bit experts are built")
        self.linear_quant_method = linear_quant_method      # "gptq" or "awq"
        self.weight_bits = weight_bits
        self.group_size = group_size
        # GPTQ 4-bit always carries zero-points, symmetric ones store 7 (+1 = 8)
        # (moe_wna16.py:73-76)
        self.has_zp = has_zp or linear_quant_method == "gptq"

    @classmethod
    def get_name(cls) -> str:
        return "moe_wna16_gcu"

    def get_quant_method(self, layer=None, prefix: str = ""):
        return MoeWNA16GCUMethod(self)


class MoeWNA16GCUMethod:
    def __init__(self, quant_config: MoeWNA16GCUConfig):
        self.quant_config = quant_config
        self.fused_experts = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), self.select_gemm_impl())

    def select_gemm_impl(self, prepare_finalize=None, moe=None):
        return TritonExpertsPad(use_int4_w4a16=True, block_shape=[0, self.quant_config.group_size])

    def process_weights_after_loading(self, layer) -> None:
        """``layer.w13_qweight`` / ``w2_qweight`` hold the stacked checkpoint
        tensors of the experts (GPTQ ``[E, K/8, N]`` or AWQ ``[E, K, N/8]``) and
        ``*_qzeros`` their packed zero-points."""
        fn = (rearrange.rearrange_uint4_int32_gptq if self.quant_config.linear_quant_method == "gptq"
              else rearrange.rearrange_uint4_int32_awq)
        for name in ("w13", "w2"):
            qw = getattr(layer, f"{name}_qweight").data
            qz = getattr(layer, f"{name}_qzeros").data if self.quant_config.has_zp else None
            w, z = fn(qw, qz)
            setattr(layer, f"{name}_qweight", Parameter(w, requires_grad=False))
            if z is not None:
                setattr(layer, f"{name}_qzeros", Parameter(z, requires_grad=False))

    def apply(self, layer, x, router_logits, top_k: int, renormalize: bool, use_grouped_topk: bool = False,
              global_num_experts: int = -1, expert_map=None, topk_group=None, num_expert_group=None,
              custom_routing_function=None, scoring_func: str = "softmax", e_score_correction_bias=None,
              activation: str = "silu", apply_router_weight_on_input: bool = False):
        topk_weights, topk_ids = select_experts(x, router_logits, top_k, use_grouped_topk, renormalize,
                                                topk_group, num_expert_group, custom_routing_function,
                                                scoring_func, e_score_correction_bias)
        has_zp = self.quant_config.has_zp
        return self.fused_experts(x, layer.w13_qweight, layer.w2_qweight, topk_weights=topk_weights,
                                  topk_ids=topk_ids, inplace=True, activation=activation,
                                  expert_map=expert_map, global_num_experts=global_num_experts,
                                  w1_scale=layer.w13_scales, w2_scale=layer.w2_scales,
                                  w1_zp=layer.w13_qzeros if has_zp else None,
                                  w2_zp=layer.w2_qzeros if has_zp else None)
