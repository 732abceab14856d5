"""MI355X-native quantized-linear kernels behind the vllm-gcu custom-op surface.

Importing the package does not load the HIP library; ``vllm_gcu_amd.kernels``
does, and fails loudly when ``libmi355q.so`` has not been built.
"""
__version__ = "0.1.0"
