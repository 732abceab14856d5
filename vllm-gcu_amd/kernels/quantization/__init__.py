"""Quantization methods of the quantized-linear path (counterpart of
vllm_gcu/kernels/quantization/__init__.py: importing the package registers
every config)."""
from . import awq, fp8, gptq, moe_wna16, w4a8, w8a8  # noqa: F401
from .utils import QUANTIZATION_METHODS, override_quantization_method  # noqa: F401
