"""Weight-only int4 / int8 MoE method on MI355X.

Mirrors ``MoeWNA16GCUConfig`` / ``MoeWNA16GCUMethod``
(vllm_gcu/kernels/quantization/moe_wna16.py:26-643): ``from_config`` reads a
GPTQ / AWQ ``quantize_config.json``; ``create_weights`` registers the stacked
per-expert checkpoint tensors with the reference's names and shapes
(moe_wna16.py:169-358); ``process_weights_after_loading`` repacks them once
(moe_wna16.py:385-563); ``select_gemm_impl`` picks the fused experts with
``use_int4_w4a16`` or ``use_int8_w8a16`` and ``block_shape=[0, group_size]``
(moe_wna16.py:574-584) and ``apply`` runs them.

Where this build differs on purpose: the reference repacks every expert on the
CPU and stores it transposed as uint8 ``[E, N, K/2]`` with float zeros
``z * s``; here the repack is one device kernel over all experts and the result
is the ``int32 [E, K/8, N]`` slab tensor with packed int4 zero-points (a layer
whose tensors are already in the reference's form still runs: the operator
recognises them, see ``_custom_ops._slab_weight``).  8-bit GPTQ experts become
``int8 [E, N, K]`` exactly as in the reference (moe_wna16.py:387-401) and take
the W8A16 grouped GEMM.
"""
from fractions import Fraction
from typing import Any, Dict, List, Optional

import torch
from torch.nn import Parameter

from ..fused_moe import select_experts
from ..modular_experts import TritonExpertsPad
from ..modular_kernel import FusedMoEModularKernel
from ..prepare_finalize import MoEPrepareAndFinalizeNoEP
from . import rearrange
from .utils import register_gcu_quantization_config


def _from_keys(config: Dict[str, Any], keys: List[str], default=...):
    for k in keys:
        if k in config:
            return config[k]
    if default is ...:
        raise ValueError(f"Cannot find any of {keys} in the model's quantization config.")
    return default


@register_gcu_quantization_config("moe_wna16_gcu")
class MoeWNA16GCUConfig:
    def __init__(self, linear_quant_method: str, weight_bits: int, group_size: int, has_zp: bool,
                 lm_head_quantized: bool = False, modules_to_not_convert: Optional[List[str]] = None,
                 full_config: Optional[Dict[str, Any]] = None):
        if linear_quant_method not in ("gptq", "awq"):
            raise ValueError("moe_wna16_gcu only support gptq and awq.")
        if weight_bits not in (4, 8) or (weight_bits == 8 and linear_quant_method != "gptq"):
            raise ValueError("Currently, only 8-bit and 4-bit weight quantization is supported for GPTQ MOE "
                             f"and 4-bit for AWQ MOE, but got {weight_bits} bits ({linear_quant_method}).")
        self.linear_quant_method = linear_quant_method
        self.weight_bits = weight_bits
        self.group_size = group_size
        # GPTQ 4-bit always carries zero-points: symmetric checkpoints store 7 (+1 = 8)
        # (moe_wna16.py:73-76)
        self.has_zp = has_zp or (linear_quant_method == "gptq" and weight_bits == 4)
        self.pack_factor = Fraction(32, weight_bits)
        self.lm_head_quantized = lm_head_quantized
        self.modules_to_not_convert = modules_to_not_convert or []
        self.full_config = full_config or {}

    @classmethod
    def get_name(cls) -> str:
        return "moe_wna16_gcu"

    @classmethod
    def get_supported_act_dtypes(cls) -> List[torch.dtype]:
        return [torch.bfloat16, torch.half]

    @classmethod
    def get_config_filenames(cls) -> List[str]:
        return ["quantize_config.json"]

    @classmethod
    def from_config(cls, config: Dict[str, Any]) -> "MoeWNA16GCUConfig":
        """moe_wna16.py:67-96."""
        method = _from_keys(config, ["quant_method"])
        bits = _from_keys(config, ["bits"])
        group_size = _from_keys(config, ["group_size"])
        lm_head = _from_keys(config, ["lm_head"], default=False)
        if method == "gptq":
            sym = _from_keys(config, ["sym"])
            has_zp = (not sym) or (sym and bits == 4)
            skip = []
        elif method == "awq":
            has_zp = _from_keys(config, ["zero_point"])
            skip = _from_keys(config, ["modules_to_not_convert"], default=None)
        else:
            raise ValueError("moe_wna16_gcu only support gptq and awq.")
        return cls(method, bits, group_size, has_zp, lm_head, skip, config)

    @classmethod
    def is_moe_wna16_gcu_compatible(cls, quant_config: Dict[str, Any]) -> bool:
        """moe_wna16.py:123-149 without the device-capability query (every MI355X qualifies)."""
        method = str(quant_config.get("quant_method", "")).lower()
        bits = quant_config.get("bits")
        if method == "gptq" and bits in (4, 8):
            return not (quant_config.get("desc_act") and not quant_config.get("static_groups", False))
        return method == "awq" and bits == 4

    @classmethod
    def override_quantization_method(cls, hf_quant_cfg, user_quant) -> Optional[str]:
        if cls.is_moe_wna16_gcu_compatible(hf_quant_cfg) and user_quant == "moe_wna16_gcu":
            return cls.get_name()
        return None

    def get_quant_method(self, layer=None, prefix: str = ""):
        return MoeWNA16GCUMethod(self)


class MoeWNA16GCUMethod:
    def __init__(self, quant_config: MoeWNA16GCUConfig):
        self.quant_config = quant_config
        self.fused_experts = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), self.select_gemm_impl())

    def select_gemm_impl(self, prepare_finalize=None, moe=None):
        bits = self.quant_config.weight_bits
        return TritonExpertsPad(use_int4_w4a16=bits == 4, use_int8_w8a16=bits == 8,
                                block_shape=[0, self.quant_config.group_size])

    def create_weights(self, layer, num_experts: int, hidden_size: int, intermediate_size_per_partition: int,
                       params_dtype: torch.dtype, **extra_weight_attrs):
        """Stacked checkpoint tensors under the reference's names (moe_wna16.py:169-358): GPTQ packs along
        K (``[E, K / pack, N]``, plus ``*_g_idx``), AWQ along N (``[E, K, N / pack]``); scales
        ``[E, K / g, N]`` (one row for ``group_size == -1``), zero-points packed along N.  Attributes
        given by the caller (``weight_loader`` ...) are attached to every parameter."""
        qc = self.quant_config
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition
        pack = int(qc.pack_factor)
        layer.quant_config = qc
        if qc.group_size != -1:
            g13, g2, strategy = H // qc.group_size, I // qc.group_size, "group"
        else:
            g13, g2, strategy = 1, 1, "channel"
        attrs = dict(extra_weight_attrs)
        attrs.update({"quant_method": strategy, "is_transposed": True})

        def reg(name, shape, dtype):
            p = Parameter(torch.empty(shape, dtype=dtype), requires_grad=False)
            for k, v in attrs.items():
                setattr(p, k, v)
            layer.register_parameter(name, p)

        if qc.linear_quant_method == "gptq":
            reg("w13_qweight", (E, H // pack, 2 * I), torch.int32)
            reg("w2_qweight", (E, I // pack, H), torch.int32)
        else:
            reg("w13_qweight", (E, H, 2 * I // pack), torch.int32)
            reg("w2_qweight", (E, I, H // pack), torch.int32)
        reg("w13_scales", (E, g13, 2 * I), params_dtype)
        reg("w2_scales", (E, g2, H), params_dtype)
        reg("w13_qzeros", (E, g13, 2 * I // pack), torch.int32)
        reg("w2_qzeros", (E, g2, H // pack), torch.int32)
        if qc.linear_quant_method == "gptq":
            reg("w13_g_idx", (E, H), torch.int32)
            reg("w2_g_idx", (E, I), torch.int32)
        layer.group_size = qc.group_size

    @staticmethod
    def _require_contiguous_g_idx(g_idx: torch.Tensor, group_size: int) -> None:
        """moe_wna16.py:438-449: groups must be runs of consecutive rows (no act-order shuffle)."""
        if group_size <= 0:
            return
        g = g_idx.reshape(g_idx.shape[0], -1).to(torch.int64)
        ok = bool((g[:, 1:] >= g[:, :-1]).all()) and bool(
            ((g[:, -1] - g[:, 0] + 1) * group_size == g.shape[1]).all())
        if not ok:
            raise AssertionError("gcu only support g_idx is continuous.")

    def process_weights_after_loading(self, layer) -> None:
        qc = self.quant_config
        if qc.linear_quant_method == "gptq" and qc.weight_bits == 8:
            # symmetric only: stored zero-points are 127 (+1 = 128); bytes become w - 128 in [E, N, K]
            # (moe_wna16.py:387-401)
            for name in ("w13", "w2"):
                qz = getattr(layer, f"{name}_qzeros").data
                if not bool((qz.view(torch.int8) == 127).all()):
                    raise AssertionError("only support sym quant")
                qw = getattr(layer, f"{name}_qweight").data
                w8 = (qw.swapaxes(1, 2).contiguous().view(torch.uint8).to(torch.int16) - 128).to(torch.int8)
                setattr(layer, f"{name}_qweight", Parameter(w8, requires_grad=False))
                if qc.group_size == -1:
                    sc = getattr(layer, f"{name}_scales").data.squeeze(1)
                    setattr(layer, f"{name}_scales", Parameter(sc, requires_grad=False))
            rearrange.kslab_parameters_(layer, ("w13_qweight", "w2_qweight"))
            return
        if qc.linear_quant_method == "gptq":
            for name in ("w13", "w2"):
                g_idx = getattr(layer, f"{name}_g_idx", None)
                if g_idx is not None and g_idx.numel():
                    self._require_contiguous_g_idx(g_idx.data, qc.group_size)
        fn = (rearrange.rearrange_uint4_int32_gptq if qc.linear_quant_method == "gptq"
              else rearrange.rearrange_uint4_int32_awq)
        for name in ("w13", "w2"):
            qw = getattr(layer, f"{name}_qweight").data
            qz = getattr(layer, f"{name}_qzeros").data if qc.has_zp else None
            w, z = fn(qw, qz)
            setattr(layer, f"{name}_qweight", Parameter(w, requires_grad=False))
            if z is not None:
                setattr(layer, f"{name}_qzeros", Parameter(z, requires_grad=False))

    def apply(self, layer, x, router_logits, top_k: int, renormalize: bool, use_grouped_topk: bool = False,
              topk_group=None, num_expert_group=None, global_num_experts: int = -1, expert_map=None,
              custom_routing_function=None, scoring_func: str = "softmax", e_score_correction_bias=None,
              apply_router_weight_on_input: bool = False, activation: str = "silu", enable_eplb: bool = False,
              expert_load_view=None, logical_to_physical_map=None, logical_replica_count=None):
        topk_weights, topk_ids = select_experts(x, router_logits, top_k, use_grouped_topk, renormalize,
                                                topk_group, num_expert_group, custom_routing_function,
                                                scoring_func, e_score_correction_bias)
        has_zp = self.quant_config.has_zp and self.quant_config.weight_bits == 4
        return self.fused_experts(x, layer.w13_qweight, layer.w2_qweight, topk_weights=topk_weights,
                                  topk_ids=topk_ids, inplace=True, activation=activation,
                                  expert_map=expert_map, global_num_experts=global_num_experts,
                                  w1_scale=layer.w13_scales, w2_scale=layer.w2_scales,
                                  w1_zp=layer.w13_qzeros if has_zp else None,
                                  w2_zp=layer.w2_qzeros if has_zp else None)
