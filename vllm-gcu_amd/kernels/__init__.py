"""Host side of the quantized-linear path: operator registration
(``_custom_ops``), MoE orchestration and the quantization method classes.
Mirrors vllm_gcu/kernels/__init__.py:3-8 of the reference."""
from . import _custom_ops  # noqa: F401  (registers torch.ops._C / _moe_C implementations)
