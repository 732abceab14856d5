"""MoE host helpers: default tile configuration, token->expert alignment,
the grouped-GEMM dispatcher and grouped top-k routing.

Mirrors vllm_gcu/kernels/fused_moe.py (get_default_config :19-37,
moe_align_block_size :40-108, invoke_fused_moe_kernel :111-231, grouped_topk
:234-267) with the same names, arguments and operator calls.
"""
from typing import Any, Dict, List, Optional, Tuple

import torch

from . import _custom_ops as ops


# Rows per expert from which the fp8 block-scaled and int8 grouped GEMMs take blocks of 128 and of 256 slots, i.e.
# the MFMA tile kernels with gathered rows instead of the weight-streaming kernel on blocks of 64 (measured on
# MI355X, us per GEMM, blocks of 64 / 128 / 256; a tile costs about the same however full it is, one of 128 slots
# about 0.8 of one of 256).  Mixtral shape, fp8, K 4096 x N 28672, 8 experts, at 48 / 64 / 96 / 128 / 192 rows per
# expert: 253 / 315 / 475 / 570 / 794 -- 221 / 233 / 251 / 357 / 420 -- 279 / 278 / 283 / 287 / 315; DeepSeek-V3 shape,
# K 7168 x N 4096, 256 experts, at 64 / 96 / 128 / 192: 2504 / 3538 / 4313 / 5962 -- 1734 / 1896 / 2576 / 4063 --
# 2177 / 2241 / 2278 / 2477.  (The library takes the tile kernels for blocks of 128 from 40 rows per expert on.)
_FP8_TILE_MIN_ROWS_PER_EXPERT = 40
_TILE_256_ROWS_PER_EXPERT = 110


def get_default_config(M: int, E: int, N: int, K: int, topk: int, dtype: Optional[str], is_marlin: bool,
                       block_shape: Optional[List[int]] = None) -> Dict[str, int]:
    """Only BLOCK_SIZE_M is consumed (as the align/GEMM block size).  The
    reference hard-codes 64 for its hardware (fused_moe.py:29-36); on MI355X the
    grouped GEMM runs 16-row MFMA tiles, so the block follows the expected rows
    per expert: 16 and 32 for decode-sized batches, 64 from there on (64-row
    tiles with two workgroups per CU were measured faster than 128-row tiles up
    to 4096 tokens on the Mixtral-8x7B layer, and they pad less)."""
    per_expert = (M * topk) / max(E, 1)
    tiles = (block_shape is not None and list(block_shape) == [128, 128]) or dtype in ("int8_w8a8", "w16a16")
    if tiles and per_expert > _FP8_TILE_MIN_ROWS_PER_EXPERT:
        # fp8 block-scaled, int8 and unquantised 16-bit experts ("w16a16": this build's name for them, the
        # reference passes None) at prefill token counts: blocks of 128 or 256 slots run the MFMA tile
        # kernels with gathered rows instead of the weight-streaming kernel
        return {"BLOCK_SIZE_M": 256 if per_expert > _TILE_256_ROWS_PER_EXPERT else 128, "BLOCK_SIZE_N": 64,
                "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}
    if per_expert <= 16:
        bm = 16
    elif per_expert <= 28:      # measured on the Mixtral-8x7B W4A16 layer: at 32 rows per expert on average
        bm = 32                 # half of the experts already need a second block of 32
    else:
        bm = 64
    return {"BLOCK_SIZE_M": bm, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int,
                         expert_map: torch.Tensor = None,
                         topk_ids_size=None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    max_num_tokens_padded = topk_ids.numel() + num_experts * (block_size - 1)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    max_num_m_blocks = max_num_tokens_padded // block_size
    expert_ids = torch.empty((max_num_m_blocks,), dtype=torch.int32, device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1), dtype=torch.int32, device=topk_ids.device)

    if topk_ids_size is not None:
        if expert_map is None:
            ops.moe_align_block_size_pad(topk_ids, topk_ids_size, num_experts, block_size, sorted_ids,
                                         expert_ids, num_tokens_post_pad)
        else:
            # the reference's VLLM_GCU_DEEPSEEK_FUSION path (fused_moe.py:72-82):
            # the expert map is applied inside the operator
            torch.ops._C.exts_moe_align_block_size(sorted_ids, expert_ids, num_tokens_post_pad, topk_ids,
                                                   topk_ids_size, expert_map, num_experts, block_size)
    else:
        if num_experts >= 224:
            ops.sgl_moe_align_block_size(topk_ids, num_experts, block_size, sorted_ids, expert_ids,
                                         num_tokens_post_pad)
        else:
            ops.moe_align_block_size(topk_ids, num_experts, block_size, sorted_ids, expert_ids,
                                     num_tokens_post_pad)
        if expert_map is not None:
            expert_ids = expert_map[expert_ids.long()].to(torch.int32)
    return sorted_ids, expert_ids, num_tokens_post_pad


def grouped_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int, renormalize: bool,
                 num_expert_group: int = 0, topk_group: int = 0, scoring_func: str = "softmax",
                 e_score_correction_bias: Optional[torch.Tensor] = None):
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    topk_weights = torch.empty((gating_output.shape[0], topk), device=gating_output.device, dtype=torch.float32)
    topk_ids = torch.empty((gating_output.shape[0], topk), device=gating_output.device, dtype=torch.int32)
    if hidden_states.numel() == 0:
        return topk_weights, topk_ids
    torch.ops._C.fused_grouped_topk(topk_weights, topk_ids, gating_output, topk, renormalize, num_expert_group,
                                    topk_group, e_score_correction_bias, scoring_func)
    return topk_weights, topk_ids


def select_experts(hidden_states: torch.Tensor, router_logits: torch.Tensor, top_k: int, use_grouped_topk: bool,
                   renormalize: bool, topk_group: Optional[int] = None, num_expert_group: Optional[int] = None,
                   custom_routing_function=None, scoring_func: str = "softmax",
                   e_score_correction_bias: Optional[torch.Tensor] = None):
    """``FusedMoE.select_experts`` as the reference's MoE methods call it
    (moe_wna16.py:612-623, w8a8.py:312-323, fp8.py:120-131): grouped top-k when
    the model uses expert groups, a custom routing function if given, else
    softmax top-k."""
    from . import _custom_ops as ops
    if use_grouped_topk:
        assert topk_group is not None and num_expert_group is not None
        return grouped_topk(hidden_states, router_logits, top_k, renormalize, num_expert_group, topk_group,
                            scoring_func, e_score_correction_bias)
    if custom_routing_function is not None:
        return custom_routing_function(hidden_states=hidden_states, gating_output=router_logits, topk=top_k,
                                       renormalize=renormalize)
    return ops.fused_topk(hidden_states, router_logits, top_k, renormalize)


def invoke_fused_moe_kernel(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, A_scale: Optional[torch.Tensor],
                            B_scale: Optional[torch.Tensor], B_zp: Optional[torch.Tensor],
                            topk_weights: torch.Tensor, topk_ids: torch.Tensor, sorted_token_ids: torch.Tensor,
                            expert_ids: torch.Tensor, num_tokens_post_padded: torch.Tensor,
                            mul_routed_weight: bool, top_k: int, config: Dict[str, Any], use_fp8_w8a8: bool,
                            use_int8_w8a8: bool, use_int8_w8a16: bool, use_int4_w4a16: bool,
                            block_shape: Optional[List[int]] = None, real_token_num=None,
                            per_channel_quant=False, bias=None, A_scale_rec=None) -> None:
    """Same dispatch rules as fused_moe.py:111-231."""
    assert topk_weights.stride(1) == 1
    assert sorted_token_ids.stride(0) == 1
    if use_fp8_w8a8 or use_int8_w8a8:
        assert B_scale is not None
    elif use_int8_w8a16 or use_int4_w4a16:
        assert B_scale is not None
        assert block_shape and block_shape[0] == 0
        assert B_zp is None or B_zp.ndim == 3
    else:
        assert A_scale is None
        assert B_scale is None
    block_size = config["BLOCK_SIZE_M"]
    if use_fp8_w8a8 or use_int8_w8a16 or use_int4_w4a16 or use_int8_w8a8:
        w4a8 = use_fp8_w8a8 and B.dtype in (torch.int8, torch.int32)   # int4 experts, fp8 activations
        if use_fp8_w8a8:
            B_zp = None
            if not w4a8:
                group_size = block_shape[1]
        elif use_int8_w8a8:
            B_zp = None
            group_size = 1
            if B_scale is not None and B_scale.ndim == 3:
                B_scale = B_scale.transpose(1, 2).contiguous()
        elif use_int4_w4a16:
            A_scale = None
            group_size = block_shape[1]
        else:
            A_scale = None
            group_size = -1
            if B_scale.dim() == 3 and B_scale.shape[1] > 1:
                group_size = B.shape[2] // B_scale.shape[1]
                assert group_size in [64, 128], \
                    f"Unsupported shape, B: {B.shape}, B_scale: {B_scale.shape} for w8a16(int8)."
        if w4a8:
            # fused_moe.py:173-195: the reciprocal input scale goes where the kernel expects A_scale
            assert A_scale_rec is not None
            torch.ops._C.fused_moe_quant_kernel_ex(C, A, B, A_scale_rec, B_scale, B_zp, None, topk_weights,
                                                   topk_ids, sorted_token_ids, expert_ids,
                                                   num_tokens_post_padded, real_token_num, mul_routed_weight,
                                                   top_k, block_size, 128, -1)
        else:
            torch.ops._C.fused_moe_quant_kernel(C, A, B, A_scale, B_scale, group_size, B_zp, topk_weights,
                                                topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                                mul_routed_weight, top_k, block_size, None, real_token_num)
    else:
        topk_weights = topk_weights.to(torch.float32)
        torch.ops._C.fused_moe_kernel(C, A, B, topk_weights, topk_ids, sorted_token_ids, expert_ids,
                                      num_tokens_post_padded, mul_routed_weight, top_k, block_size, bias)
