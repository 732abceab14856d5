"""The fused-experts sequence: align -> grouped GEMM 1 -> SiLU-gate (+ quant)
-> grouped GEMM 2 (routed weights) -> sum over slots.

Mirrors ``TritonExpertsPad`` (vllm_gcu/kernels/modular_experts.py:25-288): same
constructor flags, ``workspace_shapes`` and ``apply`` argument list, same
operator order.  Weight shapes follow this build's layouts: int4 experts are
``int32 [E, K/8, N]`` slab tensors (or the reference's ``uint8 [E, N, K/2]``),
every other mode is ``[E, N, K]``.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from .fused_moe import get_default_config, invoke_fused_moe_kernel, moe_align_block_size


@dataclass
class FusedMoEQuantConfig:
    quant_dtype: Optional[torch.dtype] = None
    per_act_token_quant: bool = False
    block_shape: Optional[list] = None

    @staticmethod
    def make(use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=False,
             per_act_token_quant=False, block_shape=None):
        qd = torch.float8_e4m3fn if use_fp8_w8a8 else (torch.int8 if use_int8_w8a8 else None)
        return FusedMoEQuantConfig(qd, per_act_token_quant, block_shape)


def moe_problem_size(a1: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk_ids: torch.Tensor,
                     int4: bool):
    """(E, M, N, K, topk) with N = 2 * intermediate; handles the int4 layouts."""
    E = w1.shape[0]
    M, K = a1.shape
    if w1.dtype == torch.int32:
        N = w1.shape[2]                      # slab tensor [E, K/8, N] (w4a16 and w4a8 experts)
    else:
        N = w1.shape[1]                      # [E, N, K] (or reference int4 [E, N, K/2])
    return E, M, N, K, topk_ids.shape[1]


class TritonExpertsPad:

    def __init__(self, use_fp8_w8a8: bool = False, use_int8_w8a8: bool = False, use_int8_w8a16: bool = False,
                 use_int4_w4a16: bool = False, per_act_token_quant: bool = False,
                 block_shape: Optional[list] = None, per_channel_quant: bool = False):
        self.quant_config = FusedMoEQuantConfig.make(use_fp8_w8a8, use_int8_w8a8, use_int8_w8a16,
                                                     use_int4_w4a16, per_act_token_quant, block_shape)
        self.use_fp8_w8a8 = use_fp8_w8a8
        self.use_int4_w4a16 = use_int4_w4a16
        self.use_int8_w8a8 = use_int8_w8a8
        self.use_int8_w8a16 = use_int8_w8a16
        self.block_shape = block_shape
        self.per_act_token_quant = per_act_token_quant

    @property
    def quant_dtype(self):
        return self.quant_config.quant_dtype

    def supports_chunking(self) -> bool:
        return True

    def supports_expert_map(self) -> bool:
        return True

    def workspace_shapes(self, a, aq, M, N, K, topk, global_num_experts, local_num_experts):
        workspace1 = (M, topk, max(N // 2, K))
        workspace2 = (M, topk, max(N, K))
        output = (M, K)
        return (workspace1, workspace2, output, a.dtype)

    def apply(self, output, hidden_states, w1, w2, topk_weights, topk_ids, activation, global_num_experts,
              expert_map, w1_scale, w2_scale, w1_zp, w2_zp, a1q_scale, a2_scale, workspace13, workspace2,
              expert_num_tokens, apply_router_weight_on_input, a1q_scale_rec=None, a2_scale_rec=None,
              static_shape: bool = False):
        assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
        assert hidden_states.dim() == 2
        assert hidden_states.dtype in [torch.float32, torch.float16, torch.bfloat16, torch.float8_e4m3fn,
                                       torch.int8]
        E, num_tokens, N, K, top_k_num = moe_problem_size(hidden_states, w1, w2, topk_ids, self.use_int4_w4a16)
        if global_num_experts == -1:
            global_num_experts = E
        unquantised = w1.dtype == hidden_states.dtype and w1.dtype in (torch.float16, torch.bfloat16)
        config = get_default_config(M=num_tokens, E=E, N=N, K=K, topk=top_k_num,
                                    dtype="int8_w8a8" if self.use_int8_w8a8 else "w16a16" if unquantised else None,
                                    is_marlin=False, block_shape=self.block_shape)
        act_dtype = workspace2.dtype
        # cache1 and cache3 share workspace2: cache1 is dead once cache2 exists
        cache1 = workspace2.reshape(-1)[:num_tokens * top_k_num * N].view(num_tokens, top_k_num, N)
        c2_dtype = self.quant_dtype if self.quant_dtype is not None else act_dtype
        c2_bytes = num_tokens * top_k_num * (N // 2) * torch.empty((), dtype=c2_dtype).element_size()
        cache2 = workspace13.reshape(-1).view(torch.uint8)[:c2_bytes].view(c2_dtype).view(
            num_tokens * top_k_num, N // 2)
        cache3 = workspace2.reshape(-1)[:num_tokens * top_k_num * K].view(num_tokens, top_k_num, K)

        sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(
            topk_ids, config["BLOCK_SIZE_M"], global_num_experts, expert_map, expert_num_tokens)

        invoke_fused_moe_kernel(hidden_states, w1, cache1, a1q_scale, w1_scale, w1_zp, topk_weights, topk_ids,
                                sorted_token_ids, expert_ids, num_tokens_post_padded, False, top_k_num, config,
                                use_fp8_w8a8=self.use_fp8_w8a8, use_int8_w8a8=self.use_int8_w8a8,
                                use_int8_w8a16=self.use_int8_w8a16, use_int4_w4a16=self.use_int4_w4a16,
                                per_channel_quant=self.per_act_token_quant, block_shape=self.block_shape,
                                real_token_num=expert_num_tokens if static_shape else None,
                                A_scale_rec=a1q_scale_rec)

        if activation != "silu":
            raise ValueError(f"Unsupported FusedMoe activation: {activation}")
        if self.use_fp8_w8a8 and w1.dtype in (torch.int8, torch.int32):
            # w4a8 experts: one static scale for the second GEMM's activations (modular_experts.py:197-211)
            assert a2_scale is not None
            torch.ops._C.silu_mul_static_fp8_quant(cache2.view(-1, top_k_num, N // 2), cache1, a2_scale,
                                                   expert_num_tokens)
        elif self.use_fp8_w8a8:
            group_size = self.block_shape[1]
            a2_scale = torch.empty((num_tokens * top_k_num, N // 2 // group_size), dtype=torch.float32,
                                   device=cache1.device)
            torch.ops._C.silu_mul_per_token_group_quant_with_size(
                cache2.view(-1, top_k_num, N // 2), a2_scale.view(-1, top_k_num, N // 2 // group_size), cache1,
                expert_num_tokens, group_size)
        elif self.use_int8_w8a8:
            tmp = torch.empty((num_tokens * top_k_num, N // 2), dtype=act_dtype, device=cache1.device)
            torch.ops._C.silu_and_mul_pad(tmp.view(-1, top_k_num, N // 2), cache1, expert_num_tokens)
            if a2_scale is not None and a2_scale.dim() == 2 and a2_scale.dtype == act_dtype \
                    and a2_scale.shape[-1] == N // 2:
                # per-expert, per-channel reciprocal input scales [E, I] (modular_experts.py:232-240 of the
                # reference): the 16-bit activations go to the grouped GEMM together with the scales
                cache2 = tmp
            elif a2_scale is not None:
                torch.ops._C.static_scaled_int8_quant(cache2, tmp, a2_scale, None)
                a2_scale = a2_scale.expand(tmp.shape[0]).contiguous() if a2_scale.numel() == 1 else a2_scale
            else:
                a2_scale = torch.empty((tmp.shape[0], 1), dtype=torch.float32, device=tmp.device)
                torch.ops._C.dynamic_scaled_int8_quant(cache2, tmp, a2_scale, None)
        else:
            torch.ops._C.silu_and_mul_pad(cache2.view(-1, top_k_num, N // 2), cache1, expert_num_tokens)

        invoke_fused_moe_kernel(cache2, w2, cache3, a2_scale, w2_scale, w2_zp, topk_weights, topk_ids,
                                sorted_token_ids, expert_ids, num_tokens_post_padded,
                                not apply_router_weight_on_input, 1, config,
                                use_fp8_w8a8=self.use_fp8_w8a8, use_int8_w8a8=self.use_int8_w8a8,
                                use_int8_w8a16=self.use_int8_w8a16, use_int4_w4a16=self.use_int4_w4a16,
                                per_channel_quant=self.per_act_token_quant, block_shape=self.block_shape,
                                real_token_num=expert_num_tokens if static_shape else None,
                                A_scale_rec=a2_scale_rec)

        torch.ops._moe_C.moe_sum_pad(output, cache3, expert_num_tokens, 1, False)
