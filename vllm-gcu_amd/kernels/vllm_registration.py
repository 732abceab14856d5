"""Registration of this build's quantization configs, methods and kernels with an importable vLLM 0.9.2.

What the reference does at import time, spread over its quantization modules, done here in one
explicit call (vLLM is not a dependency of the kernels and is never imported at module import):

* every config is registered under ``<name>_gcu`` with vLLM's ``register_quantization_config``
  (vllm_gcu/kernels/quantization/utils.py:10-13);
* HF checkpoints that say ``quant_method: gptq | awq | fp8 | w8a8 | w4a8`` are redirected to the
  ``_gcu`` variant through ``override_quantization_method`` (gptq.py:94-102, awq.py:55-63, fp8.py:37-45,
  w8a8.py:81-85, w4a8.py:109-117); ``moe_wna16_gcu`` only when the user asks for it (moe_wna16.py:150-157);
* the linear methods are listed in ``WEIGHT_LOADER_V2_SUPPORTED`` (utils.py:16-20);
* the int8 scaled-mm kernel is offered to compressed-tensors checkpoints for the out-of-tree platform
  (compressed_tensor.py:39-41) -- and for the ROCm platform, which is what an MI355X is to vLLM;
* ``get_quant_method`` tells linear layers from fused-MoE layers by vLLM's own classes
  (e.g. fp8.py:24-31) and hands skipped prefixes to ``UnquantizedLinearMethod``.

The classes of this package are plain Python classes; vLLM asserts ``isinstance`` of its own bases in
places (``FusedMoE.__init__`` wants a ``FusedMoEMethodBase``), so the registered classes are built here as
subclasses of both: ``type(name, (ours, vllm_base), {...})``.
"""
import importlib
from typing import Any, Dict, Optional

import torch

from .quantization import utils as qutils

# HF quant_method name -> (registered name, user --quantization values that still select it)
_OVERRIDES = {
    "gptq": "gptq_gcu",
    "awq": "awq_gcu",
    "fp8": "fp8_gcu",
    "w8a8": "w8a8_gcu",
    "w4a8": "w4a8_gcu",
}


def _vllm():
    """The vLLM modules the registration touches; ImportError when vLLM is absent."""
    names = {
        "quant": "vllm.model_executor.layers.quantization",
        "base": "vllm.model_executor.layers.quantization.base_config",
        "linear": "vllm.model_executor.layers.linear",
        "moe": "vllm.model_executor.layers.fused_moe.layer",
        "scaled_mm": "vllm.model_executor.layers.quantization.kernels.scaled_mm",
        "platforms": "vllm.platforms",
    }
    try:
        return {k: importlib.import_module(v) for k, v in names.items()}
    except ImportError as e:
        raise ImportError("register_with_vllm() wires the quantization configs into vLLM 0.9.2, "
                          "which is not importable here") from e


_method_classes: Dict[Any, type] = {}


def _as_vllm_method(method, base):
    """Give a method object of this package vLLM's base class too (same object, same state)."""
    if method is None or isinstance(method, base):
        return method
    key = (type(method), base)
    cls = _method_classes.get(key)
    if cls is None:
        cls = type(type(method).__name__, (type(method), base), {"__module__": type(method).__module__})
        _method_classes[key] = cls
    method.__class__ = cls
    return method


def _make_config_class(ours, v, hf_name: Optional[str]):
    QuantizationConfig = v["base"].QuantizationConfig
    LinearBase = v["linear"].LinearBase
    LinearMethodBase = v["linear"].LinearMethodBase
    Unquantized = v["linear"].UnquantizedLinearMethod
    # (install() replaces the layer class by a subclass: layers built from either are expert layers)
    FusedMoE = getattr(v["moe"].FusedMoE, "_mi355q_base", v["moe"].FusedMoE)
    FusedMoEMethodBase = v["moe"].FusedMoEMethodBase
    takes_moe = "moe" in ours.get_quant_method.__code__.co_varnames
    moe_only = ours.get_name() == "moe_wna16_gcu"

    def get_quant_method(self, layer, prefix: str = ""):
        skipped = any(name in prefix for name in (getattr(self, "modules_to_not_convert", None) or [])) or \
            any(name in prefix for name in (getattr(self, "ignored_layers", None) or []))
        if isinstance(layer, LinearBase):
            if skipped:
                return Unquantized()
            if moe_only:
                # dense layers of a moe_wna16 checkpoint take the plain GPTQ / AWQ method (moe_wna16.py:101-118)
                inner = qutils.QUANTIZATION_METHODS[f"{self.linear_quant_method}_gcu"].from_config(self.full_config)
                return _as_vllm_method(inner.get_quant_method(layer, prefix), LinearMethodBase)
            m = ours.get_quant_method(self, layer, prefix) if not takes_moe else ours.get_quant_method(self, layer, prefix, False)
            return _as_vllm_method(m, LinearMethodBase)
        if isinstance(layer, FusedMoE):
            if moe_only:
                return _as_vllm_method(ours.get_quant_method(self, layer, prefix), FusedMoEMethodBase)
            if takes_moe:
                return _as_vllm_method(ours.get_quant_method(self, layer, prefix, True), FusedMoEMethodBase)
        return None

    def override_quantization_method(cls, hf_quant_cfg, user_quant) -> Optional[str]:
        if moe_only:
            return ours.override_quantization_method.__func__(cls, hf_quant_cfg, user_quant)
        if hf_name and hf_quant_cfg.get("quant_method") == hf_name and user_quant in (hf_name, cls.get_name(), None):
            return cls.get_name()
        return None

    ns = {
        "__module__": ours.__module__,
        "get_quant_method": get_quant_method,
        "override_quantization_method": classmethod(override_quantization_method),
    }
    # the abstract class methods of vLLM's base that a plain class of this package may not spell out
    if not hasattr(ours, "get_min_capability"):
        ns["get_min_capability"] = classmethod(lambda cls: 30)
    if not hasattr(ours, "get_config_filenames"):
        ns["get_config_filenames"] = classmethod(lambda cls: ["quantize_config.json"])
    if not isinstance(ours.__dict__.get("get_supported_act_dtypes"), classmethod):
        ns["get_supported_act_dtypes"] = classmethod(lambda cls: [torch.half, torch.bfloat16])
    return type(ours.__name__, (ours, QuantizationConfig), ns)


def register_with_vllm() -> Dict[str, type]:
    """Registers every config of ``quantization.utils.QUANTIZATION_METHODS`` with vLLM and returns the
    registered classes by name.  Idempotent: a name vLLM already knows is left alone (utils.py:11-13)."""
    from . import quantization  # noqa: F401  (imports every config module: fills the registry)
    from .quantization import w8a8 as w8a8_mod
    v = _vllm()
    registered = {}
    hf_of = {gcu: hf for hf, gcu in _OVERRIDES.items()}
    for name, ours in qutils.QUANTIZATION_METHODS.items():
        if name in v["quant"].QUANTIZATION_METHODS:
            continue
        cls = _make_config_class(ours, v, hf_of.get(name))
        v["quant"].register_quantization_config(name)(cls)
        registered[name] = cls
    # linear methods whose parameters carry vLLM's v2 weight loaders (utils.py:16-20)
    supported = v["linear"].WEIGHT_LOADER_V2_SUPPORTED
    for meth in ("GPTQGCULinearMethod", "AWQGCULinearMethod", "Fp8GCULinearMethod", "W8A8LinearMethod"):
        if meth not in supported:
            supported.append(meth)
    # compressed-tensors int8: the kernel list of the platform (compressed_tensor.py:14-41)
    cutlass = importlib.import_module("vllm.model_executor.layers.quantization.kernels.scaled_mm.cutlass")

    class CompressedTensorMMLinearKernel(w8a8_mod.CompressedTensorMMLinearKernel, cutlass.CutlassScaledMMLinearKernel):
        @classmethod
        def get_min_capability(cls) -> int:
            return 30

        @classmethod
        def can_implement(cls, c):
            if not c.input_symmetric:
                return False, "CompressedTensorMMLinearKernel only supports symmetric quantization."
            return True, None

    kernels = v["scaled_mm"]._POSSIBLE_KERNELS
    enum = v["platforms"].PlatformEnum
    kernels[enum.OOT] = [CompressedTensorMMLinearKernel]
    if hasattr(enum, "ROCM"):
        kernels[enum.ROCM] = [CompressedTensorMMLinearKernel] + [k for k in kernels.get(enum.ROCM, [])
                                                                  if k.__name__ != "CompressedTensorMMLinearKernel"]
    registered["CompressedTensorMMLinearKernel"] = CompressedTensorMMLinearKernel
    # compressed-tensors int8 experts: upstream's method class with this build's kernels behind it
    # (vllm_gcu/patch/patch_0_9_2/compressed_tensor.py:12-89 replaces the class the same way)
    try:
        ctm = importlib.import_module(
            "vllm.model_executor.layers.quantization.compressed_tensors.compressed_tensors_moe")
    except ImportError:
        ctm = None
    if ctm is not None and hasattr(ctm, "CompressedTensorsW8A8Int8MoEMethod"):
        upstream = ctm.CompressedTensorsW8A8Int8MoEMethod
        if not getattr(upstream, "_mi355q", False):
            from .modular_experts import TritonExpertsPad

            def select_gemm_impl(self, prepare_finalize=None, moe=None):
                strategy = getattr(getattr(self, "input_quant", None), "strategy", "token")
                per_token = str(getattr(strategy, "value", strategy)).lower() == "token"
                return TritonExpertsPad(use_int8_w8a8=True, per_channel_quant=True, per_act_token_quant=per_token)

            gcu = type("GCUCompressedTensorsW8A8Int8MoEMethod", (upstream,),
                       {"select_gemm_impl": select_gemm_impl,
                        "apply": w8a8_mod.GCUCompressedTensorsW8A8Int8MoEMethod.apply,
                        "_mi355q": True, "__module__": w8a8_mod.__name__})
            ctm.CompressedTensorsW8A8Int8MoEMethod = gcu
            registered["GCUCompressedTensorsW8A8Int8MoEMethod"] = gcu
    return registered
