"""RMS normalisation on the CPU (numpy).  Test infrastructure only.

The reference's ``rms_norm`` / ``fused_add_rms_norm`` (csrc/src/rms_norm.cpp,
csrc/torch_bindings.cpp:254-272) call a vendor kernel whose arithmetic is not
in the repository; the contract it inherits is upstream vLLM's (v0.9.2,
``csrc/layernorm_kernels.cu``, a dependency that is not vendored), restated
here: the variance is accumulated in float32 over the row, the normalised value
is rounded to the activation type and then multiplied by the weight *in the
activation type*; with a residual, ``z = x + residual`` is formed in the
activation type first and written back as the new residual.

The fused norm + quantise operators are defined by the reference as the
sequence norm -> quantiser (vllm_gcu/compilation/fusion.py:183-330), so they
need no restatement of their own: tests compare them with that sequence.
"""
import numpy as np


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float, act) -> np.ndarray:
    """x float32 [rows, K] (values representable in the activation type),
    ``act`` rounds a float32 array to the activation type and back."""
    x = x.astype(np.float32)
    var = np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32)
    s = (np.float32(1.0) / np.sqrt(var + np.float32(eps))).astype(np.float32)
    return act(act(x * s) * weight.astype(np.float32))


def fused_add_rms_norm(x: np.ndarray, residual: np.ndarray, weight: np.ndarray, eps: float, act):
    """-> (normalised [rows, K], new residual [rows, K])."""
    z = act(x.astype(np.float32) + residual.astype(np.float32))
    return rms_norm(z, weight, eps, act), z
