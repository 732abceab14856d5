"""prepare -> fused experts -> finalize.

Mirrors ``FusedMoEModularKernel.forward`` (vllm_gcu/kernels/modular_kernel.py:42-297)
for one GPU: activation quantisation in ``prepare``, workspace allocation
(modular_kernel.py:193-198), the experts' ``apply`` and ``finalize``.
"""
from typing import Optional

import torch

from .modular_experts import moe_problem_size


class FusedMoEModularKernel(torch.nn.Module):

    def __init__(self, prepare_finalize, fused_experts):
        super().__init__()
        self.prepare_finalize = prepare_finalize
        self.fused_experts = fused_experts

    def forward(self, hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                topk_weights: torch.Tensor, topk_ids: torch.Tensor, inplace: bool = False,
                activation: str = "silu", global_num_experts: int = -1,
                expert_map: Optional[torch.Tensor] = None, w1_scale: Optional[torch.Tensor] = None,
                w2_scale: Optional[torch.Tensor] = None, w1_zp: Optional[torch.Tensor] = None,
                w2_zp: Optional[torch.Tensor] = None, a1_scale: Optional[torch.Tensor] = None,
                a2_scale: Optional[torch.Tensor] = None, apply_router_weight_on_input: bool = False,
                a1_scale_rec: Optional[torch.Tensor] = None,
                a2_scale_rec: Optional[torch.Tensor] = None) -> torch.Tensor:
        a1 = hidden_states
        # every element is written by finalize (a copy or the shared experts' output plus an add)
        output = a1 if inplace else torch.empty_like(a1)
        if a1.numel() == 0:
            return output
        fe = self.fused_experts
        E, M, N, K, top_k = moe_problem_size(a1, w1, w2, topk_ids, fe.use_int4_w4a16)
        if global_num_experts == -1:
            global_num_experts = E
        a1q, a1q_scale, expert_num_tokens, _ids, _w, shared_output = self.prepare_finalize.prepare(
            a1, a1_scale, a2_scale, topk_weights, topk_ids, global_num_experts, expert_map,
            apply_router_weight_on_input, fe.quant_config)
        ws13_shape, ws2_shape, out_shape, ws_dtype = fe.workspace_shapes(a1, a1q, M, N, K, top_k,
                                                                         global_num_experts, E)
        workspace13 = torch.empty(ws13_shape, device=a1.device, dtype=ws_dtype)
        workspace2 = torch.empty(ws2_shape, device=a1.device, dtype=ws_dtype)
        # without shared experts the experts' final sum can land in the output directly: a1 is last
        # read by the first GEMM, long before that sum is written
        direct = (getattr(self.prepare_finalize, "shared_experts", None) is None and shared_output is None
                  and tuple(out_shape) == tuple(output.shape) and output.is_contiguous())
        fused_out = output if direct else torch.empty(out_shape, device=a1.device, dtype=a1.dtype)
        fe.apply(fused_out, a1q, w1, w2, topk_weights, topk_ids, activation, global_num_experts, expert_map,
                 w1_scale, w2_scale, w1_zp, w2_zp, a1q_scale, a2_scale, workspace13, workspace2,
                 expert_num_tokens, apply_router_weight_on_input, a1_scale_rec, a2_scale_rec)
        if shared_output is not None:
            output.copy_(shared_output)
        self.prepare_finalize.finalize(output, fused_out, topk_weights, topk_ids, apply_router_weight_on_input)
        return output
