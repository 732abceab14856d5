"""Single-GPU prepare/finalize around the fused experts.

Mirrors ``MoEPrepareAndFinalizeNoEP`` (vllm_gcu/kernels/prepare_finalize.py:19-92):
``prepare`` quantises the activations the way vLLM's
``moe_kernel_quantize_input`` does for the configured mode and returns the
valid-token count as a device int32 scalar; ``finalize`` copies (or, with
shared experts, scales and adds) the fused output.  The expert-parallel
all-to-all classes of the reference are out of scope on one GPU.
"""
from typing import Optional

import torch

from . import _custom_ops as ops


def moe_kernel_quantize_input(A: torch.Tensor, A_scale: Optional[torch.Tensor], quant_dtype,
                              per_act_token_quant: bool, block_shape=None):
    if quant_dtype == torch.float8_e4m3fn:
        if block_shape is not None:
            return ops.per_token_group_quant_fp8(A, block_shape[1])
        return ops.scaled_fp8_quant(A, A_scale, use_per_token_if_dynamic=per_act_token_quant)
    if quant_dtype == torch.int8:
        q, s, _ = ops.scaled_int8_quant(A, A_scale)
        return q, s
    return A, A_scale


_TOKEN_COUNTS = {}


def _token_count(n: int, device: torch.device) -> torch.Tensor:
    """Device scalar ``int32 [1]`` holding ``n``: one per (device, value), never written again
    (a fresh ``torch.full`` per forward is a kernel launch of its own).  A cached scalar is never
    freed -- a captured graph may hold its address --; past 65536 distinct values new ones are
    simply not cached (their owner is the caller, or the capturing graph's pool)."""
    key = (device.type, device.index, int(n))
    t = _TOKEN_COUNTS.get(key)
    if t is None:
        t = torch.full((1,), int(n), dtype=torch.int32, device=device)
        if len(_TOKEN_COUNTS) < 65536:
            _TOKEN_COUNTS[key] = t
    return t


class MoEPrepareAndFinalizeNoEP:

    def __init__(self):
        self.shared_experts = None
        self.routed_scaling_factor = 1.0

    def set_shared_experts(self, shared_experts, routed_scaling_factor):
        if shared_experts is not None:
            assert routed_scaling_factor is not None
        self.shared_experts = shared_experts
        self.routed_scaling_factor = routed_scaling_factor

    def max_num_tokens_per_rank(self) -> Optional[int]:
        return None

    def topk_indices_dtype(self) -> Optional[torch.dtype]:
        return None

    def num_dispatchers(self) -> int:
        return 1

    def prepare(self, a1, a1_scale, a2_scale, topk_weights, topk_ids, num_experts, expert_map,
                apply_router_weight_on_input, quant_config):
        assert not apply_router_weight_on_input
        if a1_scale is not None and a1.dtype == a1_scale.dtype:  # w8a8-int8 static
            a1q, a1q_scale = a1, a1_scale
        else:
            a1q, a1q_scale = moe_kernel_quantize_input(a1, a1_scale, quant_config.quant_dtype,
                                                       quant_config.per_act_token_quant,
                                                       quant_config.block_shape)
        total_tokens = _token_count(a1.shape[0], a1.device)
        shared_output = None
        if self.shared_experts is not None:
            shared_output = self.shared_experts(a1)
        return a1q, a1q_scale, total_tokens, topk_ids, topk_weights, shared_output

    def finalize(self, output, fused_expert_output, topk_weights, topk_ids, apply_router_weight_on_input) -> None:
        if self.shared_experts is None:
            if fused_expert_output is not output:          # the experts may have written into it directly
                output.copy_(fused_expert_output)
        else:
            fused_expert_output.mul_(self.routed_scaling_factor)
            output.add_(fused_expert_output)
