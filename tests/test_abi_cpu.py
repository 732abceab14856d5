"""The C-ABI library loads and exports every symbol include/mi355q.h declares;
the Python operator surface registers the reference's schema strings (no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355q.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355q_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    from vllm_gcu_amd import _lib
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 8
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in mi355q.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    for n in _lib.SIGNATURES:
        assert n in names, f"{n} bound in _lib.py but not declared in mi355q.h"
    assert lib.mi355q_abi_version() == _lib.ABI_VERSION == 5


def test_argument_errors_are_reported_without_gpu():
    from vllm_gcu_amd import _lib
    lib = _lib.load()
    rc = lib.mi355q_w4a16_gemm(1, 1, 1, 1, None, 0, None, 4, 100, 128, 128, 0, None, 0, None)
    assert rc != 0
    assert b"multiples of 128" in lib.mi355q_last_error()
    rc = lib.mi355q_w4_repack(1, 9, 1, 1, 128, 128, None)
    assert rc != 0 and b"unknown source format" in lib.mi355q_last_error()
    with pytest.raises(RuntimeError, match="unknown source format"):
        _lib.check(rc, "w4_repack")


def test_ops_fail_loudly_on_cpu_tensors():
    import torch
    from vllm_gcu_amd.kernels import _custom_ops as ops
    x = torch.zeros(2, 128, dtype=torch.float16)
    w = torch.zeros(16, 128, dtype=torch.int32)
    s = torch.ones(1, 128, dtype=torch.float16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        ops.gptq_gemm_gcu(x, w, torch.empty(0, dtype=torch.int32), s, torch.empty(0, dtype=torch.int32), 4, None, 128)
