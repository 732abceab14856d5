"""W8A8 int8 linear methods on MI355X.

``W8A8LinearMethod`` mirrors vllm_gcu/kernels/quantization/w8a8.py:88-171
(static per-channel input scales, single fused output scale, ``dot_bias_quant``).
``CompressedTensorMMLinearKernel`` mirrors compressed_tensor.py:14-41 (dynamic
per-token activation scales, ``cutlass_scaled_mm``).  The reference transposes
the weight to ``[K, N]`` at load time for its hardware; the int8 MFMA consumes
K-contiguous operands, so the checkpoint's ``[N, K]`` tensor is kept and the
operator is handed its ``.t()`` view.
"""
from typing import Optional

import torch
from torch.nn import Parameter

from .. import _custom_ops as ops
from ..fused_moe import select_experts
from ..modular_experts import TritonExpertsPad
from ..modular_kernel import FusedMoEModularKernel
from ..prepare_finalize import MoEPrepareAndFinalizeNoEP
from . import rearrange
from .utils import register_gcu_quantization_config


@register_gcu_quantization_config("w8a8_gcu")
class W8A8Config:
    @classmethod
    def get_name(cls) -> str:
        return "w8a8_gcu"

    @classmethod
    def get_supported_act_dtypes(cls):
        return [torch.half, torch.bfloat16]

    @classmethod
    def from_config(cls, config):
        return cls()

    def get_quant_method(self, layer=None, prefix: str = "", moe: bool = False):
        return FusedW8A8MoEMethod(self) if moe else W8A8LinearMethod(self)


class W8A8LinearMethod:
    def __init__(self, quant_config: W8A8Config):
        self.quant_config = quant_config

    def create_weights(self, layer, input_size_per_partition, output_partition_sizes, input_size,
                       output_size, params_dtype, **extra_weight_attrs):
        layer.out_dtype = params_dtype
        out = sum(output_partition_sizes)
        layer.register_parameter("weight", Parameter(torch.empty(out, input_size_per_partition, dtype=torch.int8),
                                                     requires_grad=False))          # (N, K)
        layer.register_parameter("out_scales", Parameter(torch.ones(out, dtype=torch.float32),
                                                         requires_grad=False))      # (N)
        layer.register_parameter("in_scales", Parameter(torch.ones(input_size_per_partition, dtype=params_dtype),
                                                        requires_grad=False))       # (K)

    def process_weights_after_loading(self, layer) -> None:
        # keep [N, K] storage (the operator sees the [K, N] view), bytes re-ordered once for
        # contiguous wavefront loads where the shape allows: decode-sized batches then stream the
        # weights about twice as fast, the prefill kernel reads either order
        layer.weight = Parameter(layer.weight.data.contiguous(), requires_grad=False)
        rearrange.kslab_parameters_(layer, ("weight",))

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        if x.dtype in self.quant_config.get_supported_act_dtypes():
            x = ops.scaled_int8_quant(x, layer.in_scales)[0]
        assert x.dtype == torch.int8
        shape = list(x.shape)
        shape[-1] = int(layer.weight.shape[0])
        output = torch.empty(shape, dtype=layer.out_dtype, device=x.device)
        ops.dot_bias_quant(output, x, layer.weight.t(), layer.out_scales, bias)
        return output


class CompressedTensorMMLinearKernel:
    """Dynamic per-token int8 activations x per-channel int8 weights."""

    def process_weights_after_loading(self, layer) -> None:
        layer.weight = Parameter(layer.weight.data.contiguous(), requires_grad=False)   # [N, K]
        rearrange.kslab_parameters_(layer, ("weight",))

    def apply_weights(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        x_q, x_s, _ = ops.scaled_int8_quant(x.contiguous(), getattr(layer, "input_scale", None))
        x_2d = x_q.reshape(-1, x_q.shape[-1])
        out = ops.cutlass_scaled_mm(x_2d, layer.weight.t(), x_s, layer.weight_scale, x.dtype, bias)
        return out.reshape(x.shape[:-1] + (layer.weight.shape[0],))


class FusedW8A8MoEMethod:
    """int8 experts ``w13_weight [E, 2I, H]`` / ``w2_weight [E, H, I]`` with
    per-channel ``*_out_scales`` (w8a8.py:174-345).

    The reference's layer always carries static input scales: ``w13_in_scales [E, H]`` /
    ``w2_in_scales [E, I]`` in the activation dtype, holding the *reciprocals* of the checkpoint's
    per-expert, per-input-channel scales (its loader inverts them, w8a8.py:226-236), and hands
    them with the un-quantised activations to the grouped GEMM.  ``create_weights(...,
    static_in_scales=True)`` registers them the same way and ``load_in_scales`` does the loader's
    inversion; each (token, slot) row is then quantised with its expert's vector in front of the
    int8 GEMM (``mi355q_moe_expert_int8_quant``; the vendor kernel's own rounding is unpinned).
    Without them (the default here, an extension) activations are quantised per token on the fly."""

    def __init__(self, quant_config: W8A8Config):
        self.quant_config = quant_config
        self.fused_experts = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), self.select_gemm_impl())

    def select_gemm_impl(self, prepare_finalize=None, moe=None):
        return TritonExpertsPad(use_int8_w8a8=True, per_channel_quant=True, per_act_token_quant=True)

    def process_weights_after_loading(self, layer) -> None:
        # experts stay [E, N, K] as loaded (w8a8.py:240-262 transposes nothing either);
        # their bytes are re-ordered once for contiguous wavefront loads
        rearrange.kslab_parameters_(layer, ("w13_weight", "w2_weight"))

    def create_weights(self, layer, num_experts, hidden_size, intermediate_size_per_partition, params_dtype,
                       static_in_scales: bool = False, **extra_weight_attrs):
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition

        def reg(name, t):
            layer.register_parameter(name, Parameter(t, requires_grad=False))
        reg("w13_weight", torch.empty(E, 2 * I, H, dtype=torch.int8))
        reg("w2_weight", torch.empty(E, H, I, dtype=torch.int8))
        reg("w13_out_scales", torch.zeros(E, 2 * I, dtype=torch.float32))
        reg("w2_out_scales", torch.zeros(E, H, dtype=torch.float32))
        if static_in_scales:                       # w8a8.py:277-289
            reg("w13_in_scales", torch.ones(E, H, dtype=params_dtype))
            reg("w2_in_scales", torch.ones(E, I, dtype=params_dtype))

    @staticmethod
    def load_in_scales(param: torch.Tensor, expert_id: int, loaded_scale: torch.Tensor) -> None:
        """The reference's loader for ``*_in_scales`` (w8a8.py:226-236): the stored value is the reciprocal
        of the checkpoint's scale."""
        param.data[expert_id].copy_(loaded_scale.to(param.dtype).reciprocal())

    def apply(self, layer, x, router_logits, top_k: int, renormalize: bool, use_grouped_topk: bool = False,
              global_num_experts: int = -1, expert_map=None, topk_group=None, num_expert_group=None,
              custom_routing_function=None, scoring_func: str = "softmax", e_score_correction_bias=None,
              activation: str = "silu", apply_router_weight_on_input: bool = False):
        topk_weights, topk_ids = select_experts(x, router_logits, top_k, use_grouped_topk, renormalize,
                                                topk_group, num_expert_group, custom_routing_function,
                                                scoring_func, e_score_correction_bias)
        return self.fused_experts(x, layer.w13_weight, layer.w2_weight, topk_weights=topk_weights,
                                  topk_ids=topk_ids, inplace=True, activation=activation,
                                  global_num_experts=global_num_experts, expert_map=expert_map,
                                  w1_scale=layer.w13_out_scales, w2_scale=layer.w2_out_scales,
                                  a1_scale=getattr(layer, "w13_in_scales", None),
                                  a2_scale=getattr(layer, "w2_in_scales", None),
                                  apply_router_weight_on_input=apply_router_weight_on_input)


class GCUCompressedTensorsW8A8Int8MoEMethod(FusedW8A8MoEMethod):
    """compressed-tensors int8 experts (vllm_gcu/patch/patch_0_9_2/compressed_tensor.py:12-89,
    over upstream ``CompressedTensorsW8A8Int8MoEMethod``): the same kernels as
    ``FusedW8A8MoEMethod`` under the compressed-tensors parameter names --
    ``w13_weight [E, 2I, H]`` / ``w2_weight [E, H, I]`` int8, per-channel
    ``*_weight_scale [E, N, 1]`` fp32, ``*_input_scale`` None for per-token
    dynamic activations (``per_act_token=True``) or one static scale each."""

    def __init__(self, quant_config: Optional[W8A8Config] = None, per_act_token: bool = True):
        self.per_act_token = per_act_token
        super().__init__(quant_config or W8A8Config())

    def select_gemm_impl(self, prepare_finalize=None, moe=None):
        return TritonExpertsPad(use_int8_w8a8=True, per_channel_quant=True,
                                per_act_token_quant=self.per_act_token)

    def create_weights(self, layer, num_experts, hidden_size, intermediate_size_per_partition, params_dtype,
                       **extra_weight_attrs):
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition

        def reg(name, t):
            layer.register_parameter(name, Parameter(t, requires_grad=False))
        reg("w13_weight", torch.empty(E, 2 * I, H, dtype=torch.int8))
        reg("w2_weight", torch.empty(E, H, I, dtype=torch.int8))
        reg("w13_weight_scale", torch.ones(E, 2 * I, 1, dtype=torch.float32))
        reg("w2_weight_scale", torch.ones(E, H, 1, dtype=torch.float32))
        layer.w13_input_scale = None
        layer.w2_input_scale = None

    def apply(self, layer, x, router_logits, top_k: int, renormalize: bool, use_grouped_topk: bool = False,
              topk_group=None, num_expert_group=None, global_num_experts: int = -1, expert_map=None,
              custom_routing_function=None, scoring_func: str = "softmax", routed_scaling_factor: float = 1.0,
              e_score_correction_bias=None, apply_router_weight_on_input: bool = False, activation: str = "silu",
              enable_eplb: bool = False):
        if enable_eplb:
            raise NotImplementedError("EPLB not supported for `CompressedTensorsW8A8Int8MoEMethod` yet.")
        topk_weights, topk_ids = select_experts(x, router_logits, top_k, use_grouped_topk, renormalize,
                                                topk_group, num_expert_group, custom_routing_function,
                                                scoring_func, e_score_correction_bias)
        return self.fused_experts(x, layer.w13_weight, layer.w2_weight, topk_weights=topk_weights,
                                  topk_ids=topk_ids, inplace=True, activation=activation,
                                  global_num_experts=global_num_experts, expert_map=expert_map,
                                  w1_scale=layer.w13_weight_scale, w2_scale=layer.w2_weight_scale,
                                  a1_scale=layer.w13_input_scale, a2_scale=layer.w2_input_scale,
                                  apply_router_weight_on_input=apply_router_weight_on_input)
