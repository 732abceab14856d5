"""Registry of the quantization configs of this build.

Mirrors vllm_gcu/kernels/quantization/utils.py:10-13
(``register_gcu_quantization_config``): configs are registered under
``<name>_gcu`` and HF ``quant_method`` names are overridden to them.  vLLM is
not imported; a deployment wires ``QUANTIZATION_METHODS`` into vLLM's own
registry (``register_quantization_config`` for each entry).
"""
QUANTIZATION_METHODS = {}


def register_gcu_quantization_config(name: str):
    def deco(cls):
        QUANTIZATION_METHODS[name] = cls
        return cls
    return deco


def override_quantization_method(hf_quant_method: str, user_quant=None):
    """gptq -> gptq_gcu, awq -> awq_gcu, fp8 -> fp8_gcu, w8a8 -> w8a8_gcu
    (gptq.py:94-102, awq.py:55-63, fp8.py:37-45, w8a8.py:81-85)."""
    cand = f"{hf_quant_method}_gcu"
    return cand if cand in QUANTIZATION_METHODS else None
