"""prepare -> fused experts -> finalize.

Mirrors ``FusedMoEModularKernel.forward`` (vllm_gcu/kernels/modular_kernel.py:42-297)
for one GPU: activation quantisation in ``prepare``, workspace allocation
(modular_kernel.py:193-198), the experts' ``apply`` -- over chunks of
``VLLM_FUSED_MOE_CHUNK_SIZE`` tokens when the experts support chunking, with
workspaces sized for one chunk (modular_kernel.py:167-286) -- and ``finalize``.
"""
import os
from typing import Optional

import torch

from .modular_experts import moe_problem_size


def fused_moe_chunk_size() -> int:
    """vLLM's ``envs.VLLM_FUSED_MOE_CHUNK_SIZE`` (default 32768 tokens), read at call time."""
    return max(1, int(os.environ.get("VLLM_FUSED_MOE_CHUNK_SIZE", "32768")))


def _chunk_scales(scales: Optional[torch.Tensor], begin: int, end: int) -> Optional[torch.Tensor]:
    """Per-token scales follow their tokens into a chunk; a single scale serves every chunk."""
    if scales is None or scales.numel() == 1:
        return scales
    return scales[begin:end]


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
        chunk = fused_moe_chunk_size() if fe.supports_chunking() else M
        num_chunks = -(-M // chunk)
        if num_chunks > 1:
            # output shape from the full M, workspaces from one chunk (modular_kernel.py:176-186)
            _, _, out_shape, _ = fe.workspace_shapes(a1, a1q, M, N, K, top_k, global_num_experts, E)
            ws13_shape, ws2_shape, _, ws_dtype = fe.workspace_shapes(a1, a1q, chunk, N, K, top_k,
                                                                     global_num_experts, E)
        else:
            ws13_shape, ws2_shape, out_shape, ws_dtype = fe.workspace_shapes(a1, a1q, M, N, K, top_k,
                                                                             global_num_experts, E)
        workspace13 = torch.empty(ws13_shape, device=a1.device, dtype=ws_dtype)
        workspace2 = torch.empty(ws2_shape, device=a1.device, dtype=ws_dtype)
        # without shared experts the experts' final sum can land in the output directly: a1 is last
        # read by the first GEMM, long before that sum is written (one chunk only: a chunk's sum must
        # not overwrite rows of a1 that a later chunk still reads when the call is in place)
        direct = (num_chunks == 1 and getattr(self.prepare_finalize, "shared_experts", None) is None
                  and shared_output is None and tuple(out_shape) == tuple(output.shape) and output.is_contiguous())
        fused_out = output if direct else torch.empty(out_shape, device=a1.device, dtype=a1.dtype)
        if num_chunks == 1:
            fe.apply(fused_out, a1q, w1, w2, topk_weights, topk_ids, activation, global_num_experts, expert_map,
                     w1_scale, w2_scale, w1_zp, w2_zp, a1q_scale, a2_scale, workspace13, workspace2,
                     expert_num_tokens, apply_router_weight_on_input, a1_scale_rec, a2_scale_rec)
        else:
            m_out = out_shape[0]
            assert m_out >= M and m_out % M == 0
            out_chunk = chunk * (m_out // M)
            for c in range(num_chunks):
                b, e = c * chunk, min((c + 1) * chunk, M)
                valid = None
                if expert_num_tokens is not None:
                    # valid tokens of this chunk, on the device (the count itself is never written: it may be
                    # shared between calls or held by a captured graph)
                    valid = torch.clamp(expert_num_tokens - b, min=0, max=chunk).to(torch.int32)
                fe.apply(fused_out[c * out_chunk:min((c + 1) * out_chunk, m_out)], a1q[b:e], w1, w2,
                         topk_weights[b:e], topk_ids[b:e], activation, global_num_experts, expert_map, w1_scale,
                         w2_scale, w1_zp, w2_zp, _chunk_scales(a1q_scale, b, e), _chunk_scales(a2_scale, b, e),
                         workspace13, workspace2, valid, apply_router_weight_on_input, a1_scale_rec, a2_scale_rec)
        if shared_output is not None:
            output.copy_(shared_output)
        self.prepare_finalize.finalize(output, fused_out, topk_weights, topk_ids, apply_router_weight_on_input)
        return output
