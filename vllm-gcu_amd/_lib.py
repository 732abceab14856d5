"""ctypes binding of ``libmi355q.so`` (the C ABI declared in include/mi355q.h).

There is deliberately no fallback: if the shared library is missing or a call
fails, an exception is raised.
"""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_long, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355q.so")

F16, BF16, F32 = 0, 1, 2
ZP_NONE, ZP_PACKED, ZP_PRESCALED = 0, 1, 2
W4_SRC_GPTQ, W4_SRC_AWQ, W4_SRC_REF_KN, W4_SRC_REF_NK, W4_SRC_REF_KN_G64S = 0, 1, 2, 3, 4
Q_W4A16, Q_FP8_BLOCK, Q_INT8, Q_NONE, Q_W8A16, Q_W4_F32SCALE = 0, 1, 2, 3, 4, 5

# name -> (restype, argtypes); must list every symbol include/mi355q.h declares
SIGNATURES = {
    "mi355q_last_error": (c_char_p, []),
    "mi355q_abi_version": (c_int, []),
    "mi355q_w4_repack": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mi355q_w4_repack_zeros": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mi355q_w4_unpack": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mi355q_w4a16_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mi355q_w4a16_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                  c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mi355q_w4a16_gemm_ex": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_int,
                                     c_int, c_void_p]),
    "mi355q_w4a16_stream_plan": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mi355q_w4a16_noalloc_scratch_bytes": (c_size_t, []),
    "mi355q_w4a16_gemm_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                          c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355q_w8a8_int8_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                      c_void_p, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_int,
                                      c_void_p]),
    "mi355q_w8a8_int8_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mi355q_w8a8_int8_gemm_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                         c_void_p, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_int,
                                         c_void_p, c_size_t, c_void_p]),
    "mi355q_fp8_block_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                      c_int, c_long, c_long, c_long, c_int, c_void_p]),
    "mi355q_fp8_scaled_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                       c_int, c_int, c_long, c_long, c_long, c_int, c_void_p]),
    "mi355q_fp8_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mi355q_fp8_block_gemm_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                         c_int, c_long, c_long, c_long, c_int, c_void_p, c_size_t, c_void_p]),
    "mi355q_fp8_scaled_gemm_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                          c_int, c_int, c_long, c_long, c_long, c_int, c_void_p, c_size_t, c_void_p]),
    "mi355q_dynamic_int8_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mi355q_static_int8_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355q_silu_mul_static_int8_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_long, c_int, c_int, c_void_p]),
    "mi355q_moe_expert_int8_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                             c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355q_topk_softmax": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355q_grouped_topk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_void_p]),
    "mi355q_moe_align_block_size": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_void_p]),
    "mi355q_silu_and_mul": (c_int, [c_void_p, c_void_p, c_long, c_int, c_int, c_void_p, c_int, c_void_p]),
    "mi355q_fp8_group_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p,
                                       c_int, c_void_p]),
    "mi355q_fp8_token_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mi355q_fp8_static_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_int,
                                        c_void_p]),
    "mi355q_rms_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_long, c_int,
                                c_int, c_int, c_int, c_void_p]),
    "mi355q_fp8_to_half": (c_int, [c_void_p, c_void_p, c_long, c_int, c_void_p]),
    "mi355q_moe_sum": (c_int, [c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mi355q_moe_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mi355q_moe_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "mi355q_kslab_repack": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "mi355q_kcontig_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                    c_int, c_int, c_int, c_int, c_int, c_void_p]),
}

# must equal mi355q_abi_version() of the library (csrc/core.hip)
ABI_VERSION = 5

_lib = None


def load():
    """Load the library once; raise ImportError with build instructions if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it first with "
            "`python -c 'import __graft_entry__ as g; g.build()'` (needs hipcc)")
    lib = ctypes.CDLL(LIB_PATH)
    lib.mi355q_abi_version.restype = c_int
    if lib.mi355q_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI version {lib.mi355q_abi_version()}, this binding needs {ABI_VERSION}: "
                          "rebuild it with `python -c 'import __graft_entry__ as g; g.build()'`")
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what=""):
    if rc != 0:
        msg = load().mi355q_last_error().decode(errors="replace")
        raise RuntimeError(f"mi355q {what} failed (code {rc}): {msg}")


def call(name, *args):
    check(getattr(load(), name)(*args), name)
