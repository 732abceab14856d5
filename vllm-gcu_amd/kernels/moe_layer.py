"""Wiring of the fused-MoE modular kernel into vLLM 0.9.2's ``FusedMoE`` layer.

Mirrors vllm_gcu/patch/patch_0_9_2/moe_layer.py:21-79 and the three quantiser
hooks of vllm_gcu/patch/patch_0_9_2/utils.py:13-22.  vLLM is not imported at
module import time (it is not a dependency of the kernels); ``install()`` looks
it up and replaces the same attributes the reference replaces.  The functions
themselves only need objects with the attributes they read, so they are usable
(and tested) without vLLM.
"""
from typing import Optional

import torch

from . import _custom_ops as ops
from .modular_experts import TritonExpertsPad
from .modular_kernel import FusedMoEModularKernel
from .prepare_finalize import MoEPrepareAndFinalizeNoEP


def init_prepare_finalize(self, moe, quant_config=None):
    """``FusedMoEMethodBase.init_prepare_finalize`` as the reference replaces it
    (moe_layer.py:21-48): the modular kernel is used without expert parallelism too.
    ``moe`` is vLLM's ``FusedMoEConfig`` (read: ``use_pplx_kernels``, ``use_deepep_*_kernels``,
    ``moe_parallel_config.ep_size``).  Expert parallelism needs the all-to-all prepare/finalize
    classes, which a one-GPU build does not have: it is refused with a clear error."""
    if getattr(moe, "use_pplx_kernels", False) or getattr(moe, "use_deepep_ht_kernels", False) or \
            getattr(moe, "use_deepep_ll_kernels", False):
        raise NotImplementedError("pplx / DeepEP all-to-all kernels are not part of this build")
    self.moe = moe
    ep_size = getattr(getattr(moe, "moe_parallel_config", None), "ep_size", 1)
    if ep_size > 1:
        raise NotImplementedError("expert parallelism (ep_size > 1) needs the all-to-all prepare/finalize "
                                  "classes; this build runs on one GPU")
    prepare_finalize = MoEPrepareAndFinalizeNoEP()
    self.topk_indices_dtype = prepare_finalize.topk_indices_dtype()
    experts = self.select_gemm_impl(prepare_finalize, moe)
    self.fused_experts = FusedMoEModularKernel(prepare_finalize, experts)


def select_gemm_impl_unquant(self, prepare_finalize=None, moe=None):
    """``UnquantizedFusedMoEMethod.select_gemm_impl`` (moe_layer.py:51-56): fp16 / bf16 experts."""
    return TritonExpertsPad()


def set_shared_experts(layer) -> None:
    """What the reference's ``FusedMoE.forward_impl`` does before delegating (moe_layer.py:59-70): hand the
    layer's shared experts and routed scaling factor to the prepare/finalize object."""
    qm = getattr(layer, "quant_method", None)
    fe = getattr(qm, "fused_experts", None)
    if isinstance(fe, FusedMoEModularKernel):
        fe.prepare_finalize.set_shared_experts(getattr(layer, "shared_experts", None),
                                               getattr(layer, "routed_scaling_factor", 1.0))


def per_token_quant_int8_gcu(x: torch.Tensor):
    """patch_0_9_2/utils.py:13-15: per-token dynamic int8 quantisation -> (q, scales)."""
    x_q, scales, _ = ops.scaled_int8_quant(x)
    return x_q, scales


def install():
    """Replace, in an importable vLLM 0.9.2, the attributes the reference replaces
    (moe_layer.py:73-79, utils.py:17-22) and register the quantization configs, methods and kernels
    (``vllm_registration.register_with_vllm``; returns its dictionary of registered classes).
    Raises ImportError when vLLM is absent."""
    import importlib
    try:
        fm = importlib.import_module("vllm.model_executor.layers.fused_moe")
        fml = importlib.import_module("vllm.model_executor.layers.fused_moe.layer")
        fmu = importlib.import_module("vllm.model_executor.layers.fused_moe.utils")
        f8u = importlib.import_module("vllm.model_executor.layers.quantization.utils.fp8_utils")
    except ImportError as e:
        raise ImportError("install() wires the kernels into vLLM 0.9.2, which is not importable here") from e

    upstream_layer = getattr(fml.FusedMoE, "_mi355q_base", fml.FusedMoE)      # a second install() re-wraps the original

    class FusedMoE(upstream_layer):
        _mi355q_base = upstream_layer

        def forward_impl(self, hidden_states: torch.Tensor, router_logits: torch.Tensor):
            set_shared_experts(self)
            return super().forward_impl(hidden_states, router_logits)

    fml.FusedMoE = FusedMoE
    fm.FusedMoE = FusedMoE
    fml.FusedMoEMethodBase.init_prepare_finalize = init_prepare_finalize
    fml.UnquantizedFusedMoEMethod.select_gemm_impl = select_gemm_impl_unquant
    f8u.per_token_group_quant_fp8 = ops.per_token_group_quant_fp8
    fmu.per_token_group_quant_fp8 = ops.per_token_group_quant_fp8
    fmu.per_token_quant_int8 = per_token_quant_int8_gcu
    # quantization configs, HF-name overrides, v2 weight loaders, scaled-mm kernel list
    from .vllm_registration import register_with_vllm
    return register_with_vllm()
