"""fp8-e4m3fn linear / MoE methods on MI355X.

Mirrors ``Fp8GCULinearMethod`` / ``Fp8GCUMoEMethod`` and
``apply_w8a8_block_fp8_linear`` (vllm_gcu/kernels/quantization/fp8.py:49-205).
Block-quantised checkpoints (128 x 128 weight scales) take ``linear_quant``;
checkpoints without ``weight_block_size`` -- per-tensor or per-channel weight
scales -- take the branch the reference leaves to upstream's
``Fp8LinearMethod.apply`` (fp8.py:68-69): quantise the activations (static
scale, or one scale per token) and call ``cutlass_scaled_mm`` on fp8 operands.
"""
from typing import List, Optional

import torch

from .. import _custom_ops as ops
from ..fused_moe import select_experts
from ..modular_experts import TritonExpertsPad
from ..modular_kernel import FusedMoEModularKernel
from ..prepare_finalize import MoEPrepareAndFinalizeNoEP
from . import rearrange
from .utils import register_gcu_quantization_config


def apply_w8a8_block_fp8_linear(input: torch.Tensor, weight: torch.Tensor, block_size: List[int],
                                weight_scale: torch.Tensor, input_scale: Optional[torch.Tensor] = None,
                                bias: Optional[torch.Tensor] = None,
                                cutlass_block_fp8_supported: bool = False) -> torch.Tensor:
    output_dtype = input.dtype
    if input_scale is None:
        q_input, x_scale = ops.per_token_group_quant_fp8(input, block_size[1], dtype=torch.float8_e4m3fn,
                                                         column_major_scales=False)
    else:
        # already quantised upstream (fp8.py:189-192); the 16-bit dtype cannot be
        # recovered from the fp8 view, so the output defaults to bfloat16
        q_input, x_scale = input.view(torch.float8_e4m3fn), input_scale
        output_dtype = torch.bfloat16 if input.dtype == torch.float8_e4m3fn else input.dtype
    output_shape = [*q_input.shape[:-1], weight.shape[0]]
    output = ops.w8a8_block_fp8_matmul(q_input, weight, x_scale, weight_scale, block_size,
                                       output_dtype=output_dtype, bias=None)
    if bias is not None:
        output += bias
    return output.to(dtype=output_dtype).view(*output_shape)


@register_gcu_quantization_config("fp8_gcu")
class Fp8GCUConfig:
    def __init__(self, weight_block_size=(128, 128), activation_scheme: str = "dynamic"):
        self.weight_block_size = None if weight_block_size is None else list(weight_block_size)
        if activation_scheme not in ("dynamic", "static"):
            raise ValueError(f"fp8: unsupported activation scheme {activation_scheme!r}")
        self.activation_scheme = activation_scheme

    @classmethod
    def get_name(cls) -> str:
        return "fp8_gcu"

    @classmethod
    def from_config(cls, config):
        # upstream Fp8Config.from_config: no "weight_block_size" key means per-tensor / per-channel scales.
        # (An empty dict keeps this class's default of 128 x 128 blocks.)
        if not config:
            return cls()
        return cls(config.get("weight_block_size", None), config.get("activation_scheme", "dynamic"))

    def get_quant_method(self, layer=None, prefix: str = "", moe: bool = False):
        return Fp8GCUMoEMethod(self) if moe else Fp8GCULinearMethod(self)


class Fp8GCULinearMethod:
    """Block-quantised: ``weight`` fp8 [N, K] and ``weight_scale_inv`` f32 [N/128, K/128].
    Otherwise: ``weight`` fp8 [N, K], ``weight_scale`` f32 with one value per logical shard (merged
    projections) or per output channel, and ``input_scale`` (static scheme) or none (dynamic)."""

    def __init__(self, quant_config):
        self.quant_config = quant_config
        self.block_quant = getattr(quant_config, "weight_block_size", None) is not None

    def create_weights(self, layer, input_size_per_partition: int, output_partition_sizes: List[int],
                       input_size: int, output_size: int, params_dtype: torch.dtype, **extra_weight_attrs):
        """Checkpoint tensors as upstream vLLM 0.9.2's ``Fp8LinearMethod.create_weights`` registers them (the
        reference inherits it, fp8.py:49-70).  Block-quantised: ``weight`` fp8 ``[N, K]``, ``weight_scale_inv``
        f32 ``[ceil(N / 128), ceil(K / 128)]``, no static input scale.  Per-tensor: ``weight_scale`` f32 with one
        entry per logical shard, and with the static scheme ``input_scale`` likewise."""
        N, K = sum(output_partition_sizes), input_size_per_partition

        def reg(name, t):
            p = torch.nn.Parameter(t, requires_grad=False)
            for k, v in extra_weight_attrs.items():
                setattr(p, k, v)
            layer.register_parameter(name, p)
        reg("weight", torch.empty(N, K, dtype=torch.float8_e4m3fn))
        layer.logical_widths = list(output_partition_sizes)
        layer.orig_dtype = params_dtype
        if self.block_quant:
            bn, bk = self.quant_config.weight_block_size
            reg("weight_scale_inv", torch.empty(-(-N // bn), -(-K // bk), dtype=torch.float32))
            layer.input_scale = None
            return
        shards = len(output_partition_sizes)
        reg("weight_scale", torch.full((shards,), torch.finfo(torch.float32).min, dtype=torch.float32))
        if getattr(self.quant_config, "activation_scheme", "dynamic") == "static":
            reg("input_scale", torch.full((shards,), torch.finfo(torch.float32).min, dtype=torch.float32))
        else:
            layer.input_scale = None

    def process_weights_after_loading(self, layer) -> None:
        # the reference keeps the checkpoint tensors as they are (fp8.py:72-166);
        # here the weight bytes are re-ordered once for contiguous wavefront loads
        if not self.block_quant:
            N = layer.weight.shape[0]
            ws = layer.weight_scale.data.to(torch.float32).reshape(-1)
            widths = getattr(layer, "logical_widths", None)
            if ws.numel() not in (1, N):
                # one scale per logical shard of a merged projection.  Upstream re-quantises every shard to
                # the largest scale; the GEMM here takes a scale per output channel, so each shard keeps its
                # own scale and its own fp8 codes: nothing is rounded twice.
                if not widths or len(widths) != ws.numel() or sum(widths) != N:
                    raise RuntimeError(f"fp8: {ws.numel()} weight scales do not match the shards {widths} of {N} rows")
                ws = torch.repeat_interleave(ws, torch.tensor(widths, device=ws.device))
            layer.weight_scale = torch.nn.Parameter(ws.contiguous(), requires_grad=False)
            xs = getattr(layer, "input_scale", None)
            if xs is not None:
                # a static activation scale is one number per layer: the largest of the shards' (upstream)
                layer.input_scale = torch.nn.Parameter(xs.data.to(torch.float32).max().reshape(1), requires_grad=False)
        rearrange.kslab_parameters_(layer, ("weight",))

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None,
              x_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        if not self.block_quant:
            return self._apply_scaled_mm(layer, x, bias)
        return apply_w8a8_block_fp8_linear(input=x, weight=layer.weight,
                                           block_size=self.quant_config.weight_block_size,
                                           weight_scale=layer.weight_scale_inv,
                                           input_scale=getattr(layer, "input_scale", None) if x_scale is None else x_scale,
                                           bias=bias)

    def _apply_scaled_mm(self, layer, x, bias):
        """Upstream's ``Fp8LinearOp.apply`` on this build's operators: static scheme -> ``static_scaled_fp8_quant``
        with the layer's one input scale; dynamic -> one scale per token
        (``dynamic_per_token_scaled_fp8_quant``; the reference's per-tensor dynamic quantiser is an empty
        body, csrc/src/dynamic_scaled_fp8_quant.cpp:21-22); then ``cutlass_scaled_mm`` with the ``[K, N]``
        view of the weight and its per-tensor or per-channel scales."""
        x2 = x.reshape(-1, x.shape[-1])
        q, xs = ops.scaled_fp8_quant(x2, getattr(layer, "input_scale", None), use_per_token_if_dynamic=True)
        out = ops.cutlass_scaled_mm(q, layer.weight.t(), xs, layer.weight_scale, x.dtype, bias)
        return out.view(*x.shape[:-1], layer.weight.shape[0])


class Fp8GCUMoEMethod:
    """Experts ``w13_weight`` fp8 [E, 2I, H], ``w2_weight`` fp8 [E, H, I] with
    ``*_weight_scale_inv`` f32 block scales (fp8.py:72-166)."""

    def __init__(self, quant_config: Fp8GCUConfig):
        self.quant_config = quant_config
        self.fused_experts = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), self.select_gemm_impl())

    def select_gemm_impl(self, prepare_finalize=None, moe=None):
        return TritonExpertsPad(use_fp8_w8a8=True, block_shape=self.quant_config.weight_block_size)

    def create_weights(self, layer, num_experts: int, hidden_size: int, intermediate_size_per_partition: int,
                       params_dtype: torch.dtype, **extra_weight_attrs):
        """Block-quantised experts as upstream vLLM 0.9.2's ``Fp8MoEMethod.create_weights`` registers them
        (inherited by the reference, fp8.py:72-79): fp8 ``w13_weight [E, 2I, H]`` / ``w2_weight [E, H, I]``,
        f32 ``*_weight_scale_inv`` with one value per 128 x 128 block, dynamic activation scales."""
        bn, bk = self.quant_config.weight_block_size
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition

        def reg(name, t):
            p = torch.nn.Parameter(t, requires_grad=False)
            for k, v in extra_weight_attrs.items():
                setattr(p, k, v)
            layer.register_parameter(name, p)
        reg("w13_weight", torch.empty(E, 2 * I, H, dtype=torch.float8_e4m3fn))
        reg("w2_weight", torch.empty(E, H, I, dtype=torch.float8_e4m3fn))
        reg("w13_weight_scale_inv", torch.ones(E, 2 * (-(-I // bn)), -(-H // bk), dtype=torch.float32))
        reg("w2_weight_scale_inv", torch.ones(E, -(-H // bn), -(-I // bk), dtype=torch.float32))
        layer.w13_input_scale = None
        layer.w2_input_scale = None

    def process_weights_after_loading(self, layer) -> None:
        rearrange.kslab_parameters_(layer, ("w13_weight", "w2_weight"))

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
                                  w1_scale=layer.w13_weight_scale_inv, w2_scale=layer.w2_weight_scale_inv)
