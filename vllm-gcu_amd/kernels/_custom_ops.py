"""Operator surface of the quantized-linear path.

Registers, with ``torch.library``, implementations for the same operator names
and schemas that the reference registers in csrc/torch_bindings.cpp (library
fragments ``_C`` and ``_moe_C``) and exposes the same Python wrappers as
vllm_gcu/kernels/_custom_ops.py.  A schema is defined only when no other
extension has defined the name already (the reference's ``findSchema`` guard,
torch_bindings.cpp:114-117); the implementation is registered for the GPU
dispatch key ("CUDA" is the HIP device on PyTorch-ROCm).  Every implementation
converts tensors to raw pointers and calls the C ABI of ``libmi355q.so``.
"""
from typing import List, Optional, Tuple

import os

import torch

from .. import _lib
from . import _runtime as rt
from .quantization import rearrange

# start of the shared scratch reserved for arrival counters (they must stay zero between launches)
_WS_COUNTER_BYTES = 1 << 20

_lib.load()          # fail at import time when the HIP library is missing

_libs = {
    "_C": torch.library.Library("_C", "FRAGMENT"),
    "_moe_C": torch.library.Library("_moe_C", "FRAGMENT"),
}
# operator name -> schema text, as registered by this module
SCHEMAS = {}


def _schema_exists(qualname: str) -> bool:
    try:
        torch._C._dispatch_find_schema_or_throw(qualname, "")
        return True
    except RuntimeError:
        return False


def _register(ns: str, name: str, schema: str, fn, tags=()):
    SCHEMAS[f"{ns}::{name}"] = name + schema
    if not _schema_exists(f"{ns}::{name}"):
        _libs[ns].define(name + schema, tags=tags)
    _libs[ns].impl(name, fn, "CUDA")


# ---------------------------------------------------------------------------
# W4A16 (csrc/torch_bindings.cpp:770-788)
# ---------------------------------------------------------------------------
def _converted(t: torch.Tensor, convert):
    """Convert ``t`` once and keep the result on the tensor object itself (so
    it lives exactly as long as the source and can never be confused with a
    later allocation at the same address).  Re-converts if the source was
    written in place or re-pointed since."""
    tag = (t.data_ptr(), t._version, tuple(t.shape))
    hit = getattr(t, "_mi355q_converted", None)
    if hit is None or hit[0] != tag:
        hit = (tag, convert(t))
        t._mi355q_converted = hit
    return hit[1]


def _slab_weight(qweight: torch.Tensor, transposed: bool = False) -> torch.Tensor:
    """Return the slab-layout tensor for ``qweight``.

    int32 tensors are this build's layout already.  uint8/int8 tensors are the
    reference's half-group layout (``[K/2, N]`` dense, rearrange.py:44-56, or
    ``[E, N, K/2]`` for MoE experts with ``transposed=True``); they are
    converted on the device once, so a caller that keeps the reference's
    loader still works (at the cost of holding both copies).
    """
    if qweight.dtype == torch.int32:
        return qweight
    if qweight.dtype not in (torch.uint8, torch.int8):
        raise TypeError(f"int4 weights must be int32 (slab) or uint8/int8 (reference), got {qweight.dtype}")
    return _converted(qweight, lambda t: rearrange.from_reference_layout(t, transposed=transposed))


# Pre-scaled zero-points that are bit for bit (integer 0..15) x scale in the activation type are what the
# reference's loaders leave on a layer (rearrange.py:33-34, 103-105: ``zeros = z * scales``).  They are
# turned back into the packed integers once per tensor: w = (q - z) * s is the operator's definition
# (gptq_gemm_gcu), every kernel then takes the same reading of it, and prefill takes the pipelined loops,
# which exist for integer zero-points only.  Anything else stays as given (w = q * s - zeros).
_RECOVER_INTEGER_ZEROS = True


def _integer_zeros(zeros: torch.Tensor, scales: torch.Tensor) -> Optional[torch.Tensor]:
    """Packed int32 zero-points [..., G, N/8] if ``zeros == z.to(dtype) * scales`` bit for bit for
    integers z in 0..15 (where the scale is 0: zeros 0), else None.  Cached on ``zeros``; the check
    reads one flag back from the device, so it never runs while a graph is being captured."""
    tag = (zeros.data_ptr(), zeros._version, tuple(zeros.shape), scales.data_ptr(), scales._version)
    hit = getattr(zeros, "_mi355q_integer_zeros", None)
    if hit is not None and hit[0] == tag:
        return hit[1]
    if torch.cuda.is_current_stream_capturing():
        return None
    packed = None
    if zeros.shape == scales.shape and zeros.shape[-1] % 8 == 0:
        s32 = scales.float()
        z = torch.where(s32 != 0, torch.round(zeros.float() / s32), torch.zeros_like(s32))
        ok = (z >= 0) & (z <= 15)
        zi = torch.nan_to_num(z, nan=0.0).clamp_(0, 15)
        ok &= (zi.to(scales.dtype) * scales) == zeros
        if bool(ok.all()):
            packed = rearrange.pack_int8_zeros(zi.to(torch.uint8)).contiguous()
    zeros._mi355q_integer_zeros = (tag, packed)
    return packed


def _zero_points(zeros: Optional[torch.Tensor], act_dtype: torch.dtype, scales: Optional[torch.Tensor] = None):
    """-> (tensor or None, zeros_kind); ``scales``: the group scales as the caller holds them (in the
    activation type), for the recovery of integer zero-points from pre-scaled ones"""
    if zeros is None or zeros.numel() == 0:
        return None, _lib.ZP_NONE
    if zeros.dtype == torch.int32:
        return zeros, _lib.ZP_PACKED
    if zeros.dtype in (torch.int8, torch.uint8):
        return _converted(zeros, rearrange.pack_int8_zeros), _lib.ZP_PACKED
    if zeros.dtype == act_dtype:
        if _RECOVER_INTEGER_ZEROS and scales is not None and scales.dtype == act_dtype and scales.is_cuda:
            packed = _integer_zeros(zeros, scales)
            if packed is not None:
                return packed, _lib.ZP_PACKED
        return zeros, _lib.ZP_PRESCALED
    raise TypeError(f"zero-points of dtype {zeros.dtype} do not match activations of dtype {act_dtype}")


def w4a16_gemm(x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
               zeros: Optional[torch.Tensor], bias: Optional[torch.Tensor], group_size: int,
               split_k: int = 0, family: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = x[M, K] @ dequant(qweight) (+ bias); allocates the output
    like gptq_gemm_gcu (csrc/src/gptq_gemm_gcu.cpp:35) unless the caller brings
    a contiguous ``out [M, N]`` of the activation dtype."""
    rt.require_gpu(x, qweight, scales, zeros, bias)
    if x.dim() < 1:
        raise RuntimeError(f"w4a16_gemm expects activations [.., K], got {tuple(x.shape)}")
    qw = _slab_weight(qweight)
    lead = x.shape[:-1]
    x = x.reshape(-1, x.shape[-1])
    M, K = x.shape
    N = qw.shape[-1]
    if out is None:
        out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    elif out.dtype != x.dtype or out.numel() != M * N or not out.is_contiguous() or not out.is_cuda:
        raise RuntimeError(f"w4a16_gemm: out must be a contiguous GPU tensor of {M} x {N} {x.dtype} values")
    if x.numel() == 0:
        return out.reshape(lead + (N,))
    if qw.shape[-2] * 8 != K:
        raise RuntimeError(f"w4a16_gemm: activation K={K} does not match weight K={qw.shape[-2] * 8}")
    x = x.contiguous()
    z, zk = _zero_points(zeros, x.dtype, scales)
    scales = scales.contiguous()
    if scales.dtype != x.dtype:
        scales = scales.to(x.dtype)
    if z is not None:
        z = z.contiguous()
    if bias is not None:
        bias = bias.to(x.dtype).contiguous()
    # the kernels index these by (group row, column): sizes are checked here, not on the device
    groups = K // int(group_size) if int(group_size) > 0 else 1
    if scales.numel() != groups * N:
        raise RuntimeError(f"w4a16_gemm: scales hold {scales.numel()} values, expected {groups} x {N}")
    if z is not None and z.numel() != (groups * N // 8 if zk == _lib.ZP_PACKED else groups * N):
        raise RuntimeError(f"w4a16_gemm: zero-points of shape {tuple(z.shape)} do not fit {groups} groups x {N} columns")
    if bias is not None and bias.numel() != N:
        raise RuntimeError(f"w4a16_gemm: bias holds {bias.numel()} values, expected {N}")
    lib = _lib.load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.mi355q_w4a16_workspace_bytes(M, K, N)
        ws = rt.workspace(x.device, ws_bytes)
        _lib.check(lib.mi355q_w4a16_gemm_ex(
            out.data_ptr(), x.data_ptr(), qw.data_ptr(), scales.data_ptr(), rt.ptr(z), zk, rt.ptr(bias),
            M, K, N, int(group_size), rt.dtype_code(x.dtype), ws.data_ptr(), ws.numel(),
            int(split_k), int(family), rt.stream_ptr()), "w4a16_gemm")
    return out.reshape(lead + (N,))


def _require_trivial_g_idx(g_idx: Optional[torch.Tensor], group_size: int) -> None:
    """The kernels take groups of consecutive rows (gptq.py:141-143 rejects act-order at load time);
    an operator caller that hands over a permuting ``g_idx`` must not get silently wrong sums.  The
    check reads the tensor back once and is remembered on it."""
    if g_idx is None or g_idx.numel() == 0:
        return
    tag = (g_idx.data_ptr(), g_idx._version, int(group_size))
    if getattr(g_idx, "_mi355q_trivial", None) == tag:
        return
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("gptq_gemm_gcu: this g_idx has not been checked yet and the check reads it back to the "
                           "host; call the operator once with it before capturing a graph")
    K = g_idx.numel()
    gs = int(group_size) if group_size > 0 else K
    want = torch.arange(K, device=g_idx.device, dtype=g_idx.dtype) // gs
    if not bool(torch.equal(g_idx.reshape(-1), want)):
        raise RuntimeError("gptq_gemm_gcu: act-order checkpoints (a g_idx that is not k // group_size) are "
                           "not supported")
    g_idx._mi355q_trivial = tag


def _gptq_gemm_gcu_impl(a, b_q_weight, b_gptq_qzeros, b_gptq_scales, b_g_idx, bit, bias, group_size):
    _require_trivial_g_idx(b_g_idx, group_size)
    if bit != 4:
        raise RuntimeError("gptq_gemm_gcu: only bit == 4 takes this operator "
                           "(8-bit goes through weight_only_quant)")
    return w4a16_gemm(a, b_q_weight, b_gptq_scales, b_gptq_qzeros, bias, group_size)


def _awq_gemm_gcu_impl(_in_feats, _kernel, _scaling_factors, _zeros, split_k_iters, bias, group_size):
    return w4a16_gemm(_in_feats, _kernel, _scaling_factors, _zeros, bias, group_size)


_register("_C", "gptq_gemm_gcu",
          "(Tensor a, Tensor b_q_weight, Tensor b_gptq_qzeros, Tensor b_gptq_scales, Tensor b_g_idx, "
          "int bit, Tensor? bias, int group_size) -> Tensor", _gptq_gemm_gcu_impl)
_register("_C", "awq_gemm_gcu",
          "(Tensor _in_feats, Tensor _kernel, Tensor _scaling_factors, Tensor _zeros, "
          "SymInt split_k_iters, Tensor? bias, int group_size) -> Tensor", _awq_gemm_gcu_impl)


# awq (vllm_gcu/kernels/_custom_ops.py:213-238; the reference's parameter names
# for scales / zeros are swapped relative to the schema, positions are kept)
def awq_gemm_gcu(input: torch.Tensor, qweight: torch.Tensor, qzeros: torch.Tensor,
                 scales: torch.Tensor, split_k_iters: int, bias=None, group_size=128) -> torch.Tensor:
    return torch.ops._C.awq_gemm_gcu(input, qweight, qzeros, scales, split_k_iters, bias, group_size)


@torch.library.register_fake("_C::awq_gemm_gcu")
def _awq_gemm_gcu_fake(input, qweight, qzeros, scales, split_k_iters, bias=None, group_size=128):
    out_shape = input.shape[:-1] + (qweight.shape[-1],)
    return torch.empty(out_shape, dtype=input.dtype, device=input.device)


# gptq (vllm_gcu/kernels/_custom_ops.py:242-293)
def gptq_gemm_gcu(a: torch.Tensor, b_q_weight: torch.Tensor, b_gptq_qzeros: torch.Tensor,
                  b_gptq_scales: torch.Tensor, b_g_idx: torch.Tensor, bit: int, bias=None,
                  group_size=128) -> torch.Tensor:
    assert bit in [4, 8]
    if bit == 4:
        out_shape = a.shape[:-1] + (b_q_weight.shape[-1],)
        reshaped_a = a.reshape(-1, a.shape[-1])
        output = torch.ops._C.gptq_gemm_gcu(reshaped_a, b_q_weight, b_gptq_qzeros, b_gptq_scales,
                                            b_g_idx, bit, bias, group_size)
        return output.reshape(out_shape)
    out_shape = a.shape[:-1] + (b_q_weight.shape[0],)
    output = torch.empty(out_shape, dtype=a.dtype, device=a.device)
    torch.ops._C.weight_only_quant(output, a, b_q_weight, bias, b_gptq_scales, group_size)
    return output


@torch.library.register_fake("_C::gptq_gemm_gcu")
def _gptq_gemm_gcu_fake(a, b_q_weight, b_gptq_qzeros, b_gptq_scales, b_g_idx, bit, bias=None,
                        group_size=128):
    if bit == 4:
        out_shape = a.shape[:-1] + (b_q_weight.shape[-1],)
    else:
        out_shape = a.shape[:-1] + (b_q_weight.shape[0],)
    return torch.empty(out_shape, dtype=a.dtype, device=a.device)


# ---------------------------------------------------------------------------
# W8A8 int8 (csrc/torch_bindings.cpp:734-766, 1002-1019)
# ---------------------------------------------------------------------------
_INT8_STREAM_MAX_M = 64      # measured on MI355X (K 8192, N 28672): 40-51 us against 90 us for the MFMA tile kernel


def _int8_stream_rows(K: int, N: int) -> int:
    """Up to how many rows the weight-streaming kernel takes a kslab layer (measured on MI355X, us,
    streaming / MFMA tile kernel).  The streaming kernel gives a layer of few columns 32 or 16 columns per
    workgroup, so every CU streams a share; the tile kernel's wavefronts without rows only copy, and on
    layers of at most 128 column tiles it cuts K into ranges that fill the chip.  The streaming kernel's
    time grows with the rows (in steps at 17, 33), the split tile kernel's hardly does: they cross at
    25..32 rows behind a very long K -- 28672 x 8192: M = 24 45.4 / 50.5, M = 32 51.5 / 50.7, M = 64 67.1 / 49.7;
    at 33..40 where K >= 2 N -- 16384 x 7168: M = 32 26.2 / 29.6, M = 40 31.0 / 30.3; 14336 x 4096: M = 32 19.5 / 20.1,
    M = 40 24.4 / 20.2; at 41..48 for other K >= 7168 -- 7168 x 4096: M = 40 14.9 / 15.9, M = 48 16.2 / 16.1;
    8192 x 8192: M = 48 19.5 / 21.3, M = 64 23.0 / 22.0; on wide layers (128 column tiles or more, no split)
    -- 8192 x 28672: M = 40 49.8 / 52.3, M = 48 51.9 / 49.1; a short K stays with the streaming kernel --
    4096 x 4096: M = 64 13.4 / 15.6."""
    top = _INT8_STREAM_MAX_M
    if N % 128 != 0:
        return top
    if N >= 128 * 128:
        return top * 5 // 8
    if K >= 24576:
        return top * 3 // 8
    if K >= 2 * N and K >= 7168:
        return top // 2
    if K >= 7168:
        return top * 5 // 8
    return top


def _int8_weight_nk(weight: torch.Tensor):
    """-> (tensor whose memory is [N, K] K-contiguous, row stride in bytes).

    ``weight`` is the operator's ``[K, N]`` argument.  The compressed-tensors
    path hands over ``w.t()`` of an ``[N, K]`` checkpoint tensor (strides
    ``(1, K)``, csrc/torch_bindings.cpp:1013-1017 tags the op flexible_layout),
    which already is the layout the int8 MFMA consumes.  A physically ``[K, N]``
    tensor (w8a8.py:152-155 transposes at load time) is transposed back once.
    """
    if weight.dim() != 2 or weight.dtype != torch.int8:
        raise RuntimeError(f"int8 weight must be a 2-D int8 tensor, got {weight.dtype} {tuple(weight.shape)}")
    if rearrange.is_kslab(weight):
        # bytes re-ordered at load time (rearrange.to_kslab): row stride 0 tells the library so
        return weight, 0
    if weight.stride(0) == 1 and weight.stride(1) >= weight.shape[0] and weight.stride(1) % 16 == 0:
        return weight, weight.stride(1)
    wt = _converted(weight, lambda t: t.t().contiguous())
    return wt, wt.stride(0)


def _scaled_int8_mm(out, x, weight, x_scale, w_scale, bias, acc_out=None):
    rt.require_gpu(out, x, weight, x_scale, w_scale, bias)
    if x.numel() == 0:
        return
    if x.dtype != torch.int8:
        raise RuntimeError(f"scaled int8 matmul needs int8 activations, got {x.dtype}")
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or x2.stride(0) % 16 != 0:
        x2 = x2.contiguous()
    M, K = x2.shape
    if weight.shape[0] != K:
        raise RuntimeError(f"weight is {tuple(weight.shape)} but activations have K={K}")
    N = weight.shape[1]
    w, ldw = _int8_weight_nk(weight)
    out2 = out.reshape(-1, N)
    if out2.data_ptr() != out.data_ptr() or out2.stride(-1) != 1:
        raise RuntimeError("output must be a dense [.., N] tensor")
    xs = ws = None
    xs_row = ws_col = 0
    if x_scale is not None:
        xs = x_scale.to(torch.float32).reshape(-1).contiguous()
        xs_row = int(xs.numel() > 1)
        if xs_row and xs.numel() != M:
            raise RuntimeError(f"x_scale has {xs.numel()} entries for M={M}")
    if w_scale is not None:
        ws = w_scale.to(torch.float32).reshape(-1).contiguous()
        ws_col = int(ws.numel() > 1)
        if ws_col and ws.numel() != N:
            raise RuntimeError(f"w_scale has {ws.numel()} entries for N={N}")
    bias_f32 = 0
    if bias is not None:
        bias_f32 = int(bias.dtype == torch.float32)
        if not bias_f32 and bias.dtype != out.dtype:
            bias = bias.to(torch.float32)
            bias_f32 = 1
        bias = bias.contiguous()
    stream_rows = _int8_stream_rows(K, N)
    # (row-major [N, K] weights: the tile kernel with its K ranges is level with the streaming kernel on
    # large layers -- 8192 x 28672 at M = 16: 54 against 58 us -- and behind it on small ones up to 32
    # rows: 4096 x 4096 at M = 16: 13.8 against 7.7 us)
    small_row_major = ldw == K and M <= stream_rows // 2 and K * N <= (1 << 25) and N % 4 == 0 and K % 128 == 0
    if (ldw == 0 and M <= stream_rows or small_row_major) and acc_out is None and ws_col \
            and (xs is None or xs_row or M == 1) \
            and not bias_f32 and out.dtype in (torch.float16, torch.bfloat16) and x2.is_contiguous() \
            and out2.stride(0) == N:
        # decode-sized M on kslab weights: the weight-streaming kernel (same int32 sums, same
        # epilogue order: bit-identical results) reads them about twice as fast
        with torch.cuda.device(x.device):
            _lib.call("mi355q_kcontig_gemm", out2.data_ptr(), x2.data_ptr(), w.data_ptr(), rt.ptr(xs), ws.data_ptr(),
                      rt.ptr(bias), _lib.Q_INT8, 0, M, K, N, _lib.F16, rt.dtype_code(out.dtype),
                      1 if ldw == 0 else 0, rt.stream_ptr())
        return
    with torch.cuda.device(x.device):
        # (few output tiles behind a long K: K ranges side by side through the stream's workspace, bit-identical)
        need = _lib.load().mi355q_w8a8_int8_workspace_bytes(M, N, K)
        wsp = rt.workspace(x.device, need) if need else None
        _lib.call("mi355q_w8a8_int8_gemm_ws", out2.data_ptr(), rt.ptr(acc_out), x2.data_ptr(), w.data_ptr(),
                  rt.ptr(xs), xs_row, rt.ptr(ws), ws_col, rt.ptr(bias), bias_f32, M, N, K,
                  x2.stride(0), ldw, out2.stride(0), rt.dtype_code(out.dtype), rt.ptr(wsp),
                  0 if wsp is None else wsp.numel(), rt.stream_ptr())


def _scaled_fp8_mm(out, x, weight, x_scale, w_scale, bias):
    """fp8-e4m3fn operands through ``cutlass_scaled_mm`` (cutlass_scaled_mm.cpp:12-36 forwards any dtype;
    the non-block branch of the fp8 linear method ends here, kernels/quantization/fp8.py:68-69):
    ``out = (x @ weight) * x_scale * w_scale (+ bias)`` with ``x_scale`` one value or one per row and
    ``w_scale`` one value or one per output channel, fp32 accumulation."""
    rt.require_gpu(out, x, weight, x_scale, w_scale, bias)
    if x.numel() == 0:
        return
    if weight.dtype != torch.float8_e4m3fn or weight.dim() != 2:
        raise RuntimeError(f"fp8 scaled matmul needs a 2-D float8_e4m3fn weight, got {weight.dtype} {tuple(weight.shape)}")
    if out.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"fp8 scaled matmul writes float16 or bfloat16, got {out.dtype}")
    if x_scale is None or w_scale is None:
        raise RuntimeError("fp8 scaled matmul needs both scales")
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or x2.stride(0) % 16 != 0:
        x2 = x2.contiguous()
    M, K = x2.shape
    if weight.shape[0] != K:
        raise RuntimeError(f"weight is {tuple(weight.shape)} but activations have K={K}")
    N = weight.shape[1]
    out2 = out.reshape(-1, N)
    if out2.data_ptr() != out.data_ptr() or out2.stride(-1) != 1:
        raise RuntimeError("output must be a dense [.., N] tensor")
    # the operator's weight argument is the [K, N] view of an [N, K] K-contiguous tensor (or kslab bytes)
    if rearrange.is_kslab(weight):
        w, ldw = weight, 0
    elif weight.stride(0) == 1 and weight.stride(1) >= K:
        w, ldw = weight, weight.stride(1)
        if _AUTO_KSLAB and ldw == K and rearrange.kslab_eligible(weight.t()):
            w, ldw = _converted(weight, lambda t: rearrange.to_kslab(t.t())), 0
    else:
        w = _converted(weight, lambda t: t.t().contiguous())
        ldw = w.stride(0)
    xs = x_scale.to(torch.float32).reshape(-1).contiguous()
    ws = w_scale.to(torch.float32).reshape(-1).contiguous()
    if xs.numel() not in (1, M):
        raise RuntimeError(f"x_scale has {xs.numel()} entries for M={M}")
    if ws.numel() not in (1, N):
        raise RuntimeError(f"w_scale has {ws.numel()} entries for N={N}")
    if bias is not None:
        bias = bias.to(out.dtype).contiguous()
        if bias.numel() != N:
            raise RuntimeError(f"bias has {bias.numel()} entries for N={N}")
    with torch.cuda.device(x.device):
        # (few output tiles behind a long K: K ranges side by side through the stream's workspace)
        need = _lib.load().mi355q_fp8_gemm_workspace_bytes(M, N, K)
        wsp = rt.workspace(x.device, need) if need else None
        _lib.call("mi355q_fp8_scaled_gemm_ws", out2.data_ptr(), x2.data_ptr(), w.data_ptr(), xs.data_ptr(),
                  int(xs.numel() > 1), ws.data_ptr(), int(ws.numel() > 1), rt.ptr(bias), M, N, K,
                  x2.stride(0), ldw, out2.stride(0), rt.dtype_code(out.dtype), rt.ptr(wsp),
                  0 if wsp is None else wsp.numel(), rt.stream_ptr())


def _cutlass_scaled_mm_impl(out, x, weight, x_scale, w_scale, bias):
    if x.dtype == torch.float8_e4m3fn:
        _scaled_fp8_mm(out, x, weight, x_scale, w_scale, bias)
    else:
        _scaled_int8_mm(out, x, weight, x_scale, w_scale, bias)


def _dot_bias_quant_impl(out, lhs, rhs, scale, bias):
    # single scale[N]: the activation scale is pre-folded (w8a8.py:157-171).  The reference
    # promotes the bias to fp32 before adding it (dot_bias_quant.cpp:19-21); the kernels read a
    # bias of the output type and widen each element, which is the same sum
    _scaled_int8_mm(out, lhs, rhs, None, scale, bias)


def _dynamic_scaled_int8_quant_impl(output, input, scales, azp):
    rt.require_gpu(output, input, scales)
    if azp is not None:
        raise RuntimeError("dynamic_scaled_int8_quant: asymmetric quantisation (azp) is not supported")
    if input.numel() == 0:
        return
    x = input.contiguous()
    K = x.shape[-1]
    M = x.numel() // K
    if not output.is_contiguous() or not scales.is_contiguous() or scales.dtype != torch.float32:
        raise RuntimeError("dynamic_scaled_int8_quant: output and fp32 scales must be contiguous")
    with torch.cuda.device(x.device):
        _lib.call("mi355q_dynamic_int8_quant", output.data_ptr(), scales.data_ptr(), x.data_ptr(), M, K,
                  rt.dtype_code(x.dtype), 0, rt.stream_ptr())


def _static_scaled_int8_quant_impl(result, input, scale, azp):
    rt.require_gpu(result, input, scale)
    if input.numel() == 0:
        return
    x = input.contiguous()
    K = x.shape[-1]
    M = x.numel() // K
    sc = scale.to(torch.float32).reshape(-1).contiguous()
    if sc.numel() not in (1, K):
        raise RuntimeError(f"static_scaled_int8_quant: scale must have 1 or K={K} entries, got {sc.numel()}")
    with torch.cuda.device(x.device):
        _lib.call("mi355q_static_int8_quant", result.data_ptr(), x.data_ptr(), sc.data_ptr(),
                  int(sc.numel() > 1), M, K, rt.dtype_code(x.dtype), rt.stream_ptr())


_register("_C", "cutlass_scaled_mm",
          "(Tensor! out, Tensor x, Tensor weight, Tensor x_scale, Tensor w_scale, Tensor? bias) -> ()",
          _cutlass_scaled_mm_impl, tags=(torch.Tag.flexible_layout,))
_register("_C", "dot_bias_quant", "(Tensor! out, Tensor lhs, Tensor rhs, Tensor scale, Tensor? bias) -> ()",
          _dot_bias_quant_impl)
# `azp` is a plain Tensor in the reference's schema and Python passes None for
# it (modular_experts.py:246); when this module owns the schema it is optional
_register("_C", "dynamic_scaled_int8_quant",
          "(Tensor! output, Tensor input, Tensor! scales, Tensor? azp) -> ()", _dynamic_scaled_int8_quant_impl)
_register("_C", "static_scaled_int8_quant",
          "(Tensor! result, Tensor input, Tensor scale, Tensor? azp) -> ()", _static_scaled_int8_quant_impl)


def scaled_int8_quant(input: torch.Tensor, scale: Optional[torch.Tensor] = None,
                      azp: Optional[torch.Tensor] = None, symmetric: bool = True):
    """vLLM's ``ops.scaled_int8_quant`` as the reference calls it (w8a8.py:164;
    patch/patch_0_9_2/utils.py:13-15): static when ``scale`` is given, else
    dynamic per token.  Returns ``(q int8, scales f32 [.., 1], azp None)``."""
    output = torch.empty_like(input, dtype=torch.int8)
    if scale is not None:
        torch.ops._C.static_scaled_int8_quant(output, input, scale, azp)
        return output, scale, azp
    scales = torch.empty((input.numel() // input.shape[-1], 1), device=input.device, dtype=torch.float32)
    torch.ops._C.dynamic_scaled_int8_quant(output, input.contiguous(), scales, None)
    return output, scales, None


def cutlass_scaled_mm(a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                      out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """vLLM's ``ops.cutlass_scaled_mm`` (compressed_tensor.py:32-36): allocates
    ``out [M, N]`` and calls the operator."""
    out = torch.empty((a.shape[0], b.shape[1]), dtype=out_dtype, device=a.device)
    torch.ops._C.cutlass_scaled_mm(out, a, b, scale_a, scale_b, bias)
    return out


def dot_bias_quant(out: torch.Tensor, lhs: torch.Tensor, rhs: torch.Tensor, scale: torch.Tensor,
                   bias: Optional[torch.Tensor] = None) -> None:
    torch.ops._C.dot_bias_quant(out, lhs, rhs, scale, bias)


def int8_gemm_accumulators(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """Raw int32 accumulators of the int8 GEMM (parity/debug helper)."""
    acc = torch.empty((x.shape[0], weight.shape[1]), dtype=torch.int32, device=x.device)
    out = torch.empty((x.shape[0], weight.shape[1]), dtype=torch.float32, device=x.device)
    _scaled_int8_mm(out, x, weight, None, None, None, acc_out=acc)
    return acc


# ---------------------------------------------------------------------------
# MoE routing / align (csrc/torch_bindings.cpp:803-809, 1052-1063, 1178-1189,
# 1390-1431)
# ---------------------------------------------------------------------------
def _topk_softmax_impl(topk_weights, topk_indices, token_expert_indices, gating_output):
    rt.require_gpu(topk_weights, topk_indices, token_expert_indices, gating_output)
    if gating_output.numel() == 0:
        return
    g = gating_output.contiguous()
    M, E = g.shape
    k = topk_weights.shape[-1]
    if topk_weights.dtype != torch.float32 or topk_indices.dtype != torch.int32:
        raise RuntimeError("topk_softmax: topk_weights must be float32 and topk_indices int32")
    if not (topk_weights.is_contiguous() and topk_indices.is_contiguous()):
        raise RuntimeError("topk_softmax: outputs must be contiguous")
    tei = token_expert_indices
    if tei is not None and (tei.dtype != torch.int32 or not tei.is_contiguous()):
        raise RuntimeError("topk_softmax: token_expert_indices must be contiguous int32")
    with torch.cuda.device(g.device):
        _lib.call("mi355q_topk_softmax", topk_weights.data_ptr(), topk_indices.data_ptr(), rt.ptr(tei),
                  g.data_ptr(), M, E, k, 0, rt.dtype_code(g.dtype), rt.stream_ptr())


def _fused_grouped_topk_impl(topk_weights, topk_ids, gating_output, topk, renormalize, num_expert_group,
                             topk_group, e_score_correction_bias, scoring_func):
    rt.require_gpu(topk_weights, topk_ids, gating_output, e_score_correction_bias)
    if gating_output.numel() == 0:
        return
    if scoring_func not in ("softmax", "sigmoid"):
        raise RuntimeError(f"fused_grouped_topk: unsupported scoring function {scoring_func!r}")
    g = gating_output.contiguous()
    M, E = g.shape
    bias = e_score_correction_bias
    if bias is not None:
        bias = bias.to(torch.float32).contiguous()
    if topk_weights.dtype != torch.float32 or topk_ids.dtype != torch.int32:
        raise RuntimeError("fused_grouped_topk: topk_weights must be float32 and topk_ids int32")
    with torch.cuda.device(g.device):
        _lib.call("mi355q_grouped_topk", topk_weights.data_ptr(), topk_ids.data_ptr(), g.data_ptr(),
                  rt.ptr(bias), M, E, int(topk), int(bool(renormalize)), int(num_expert_group),
                  int(topk_group), int(scoring_func == "sigmoid"), rt.dtype_code(g.dtype), rt.stream_ptr())


def _align(topk_ids, valid_rows, num_experts, block_size, expert_map, sorted_token_ids, experts_ids,
           num_tokens_post_pad):
    rt.require_gpu(topk_ids, valid_rows, expert_map, sorted_token_ids, experts_ids, num_tokens_post_pad)
    ids = topk_ids.contiguous()
    if ids.dtype not in (torch.int32, torch.int64):
        raise RuntimeError(f"moe_align_block_size: topk_ids must be int32 or int64, got {ids.dtype}")
    numel = ids.numel()
    top = ids.shape[-1] if ids.dim() > 1 else 1
    cap = numel + num_experts * (block_size - 1)
    if sorted_token_ids.numel() < cap or experts_ids.numel() < cap // block_size:
        raise RuntimeError("moe_align_block_size: output buffers are smaller than "
                           "numel + num_experts * (block_size - 1)")
    for t in (sorted_token_ids, experts_ids, num_tokens_post_pad):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("moe_align_block_size: outputs must be contiguous int32")
    if valid_rows is not None and valid_rows.dtype != torch.int32:
        valid_rows = valid_rows.to(torch.int32)
    if expert_map is not None:
        expert_map = expert_map.to(torch.int32).contiguous()
    with torch.cuda.device(ids.device):
        _lib.call("mi355q_moe_align_block_size", ids.data_ptr(), int(ids.dtype == torch.int64), numel, top,
                  rt.ptr(valid_rows), int(num_experts), int(block_size), rt.ptr(expert_map),
                  sorted_token_ids.data_ptr(), experts_ids.data_ptr(), num_tokens_post_pad.data_ptr(),
                  rt.stream_ptr())


def _moe_align_block_size_impl(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                               num_tokens_post_pad):
    _align(topk_ids, None, num_experts, block_size, None, sorted_token_ids, experts_ids, num_tokens_post_pad)


def _moe_align_block_size_pad_impl(topk_ids, topk_ids_size, num_experts, block_size, sorted_token_ids,
                                   experts_ids, num_tokens_post_pad):
    _align(topk_ids, topk_ids_size, num_experts, block_size, None, sorted_token_ids, experts_ids,
           num_tokens_post_pad)


def _exts_moe_align_block_size_impl(sorted_token_ids, experts_ids, num_tokens_post_pad, topk_ids,
                                    real_token_num, expert_map, num_experts, block_size):
    _align(topk_ids, real_token_num, num_experts, block_size, expert_map, sorted_token_ids, experts_ids,
           num_tokens_post_pad)


_register("_moe_C", "topk_softmax",
          "(Tensor! topk_weights, Tensor! topk_indices, Tensor! token_expert_indices, Tensor gating_output) -> ()",
          _topk_softmax_impl)
# e_score_correction_bias is a plain Tensor in the reference and Python passes
# None (fused_moe.py:256-266); optional where this module owns the schema
_register("_C", "fused_grouped_topk",
          "(Tensor! topk_weights, Tensor! topk_ids, Tensor gating_output, SymInt topk, bool renormalize, "
          "SymInt num_expert_group, SymInt topk_group, Tensor? e_score_correction_bias, str scoring_func) -> ()",
          _fused_grouped_topk_impl)
_register("_moe_C", "moe_align_block_size",
          "(Tensor topk_ids, int num_experts, int block_size, Tensor! sorted_token_ids, Tensor! experts_ids, "
          "Tensor! num_tokens_post_pad) -> ()", _moe_align_block_size_impl)
_register("_moe_C", "sgl_moe_align_block_size",
          "(Tensor topk_ids, int num_experts, int block_size, Tensor! sorted_token_ids, Tensor! experts_ids, "
          "Tensor! num_tokens_post_pad) -> ()", _moe_align_block_size_impl)
# registered from a C++ function pointer in the reference, hence positional-only
# callers (torch_bindings.cpp:803-809, moe_align_block_size_pad.cpp:43-47)
_register("_C", "moe_align_block_size_pad",
          "(Tensor topk_ids, Tensor topk_ids_size, int num_experts, int block_size, Tensor! sorted_token_ids, "
          "Tensor! experts_ids, Tensor! num_tokens_post_pad) -> ()", _moe_align_block_size_pad_impl)
_register("_C", "exts_moe_align_block_size",
          "(Tensor(a!) sorted_token_ids, Tensor(a!) experts_ids, Tensor(a!) num_tokens_post_pad, Tensor topk_ids, "
          "Tensor real_token_num, Tensor expert_map, int num_experts, int block_size) -> ()",
          _exts_moe_align_block_size_impl)


def topk_softmax(topk_weights, topk_ids, token_expert_indices, gating_output) -> None:
    torch.ops._moe_C.topk_softmax(topk_weights, topk_ids, token_expert_indices, gating_output)


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int, renormalize: bool):
    """vLLM's ``fused_topk`` as used by ``FusedMoE.select_experts``
    (moe_wna16.py:612-623): softmax -> top-k (descending) -> optional renorm."""
    M = gating_output.shape[0]
    topk_weights = torch.empty(M, topk, dtype=torch.float32, device=gating_output.device)
    topk_ids = torch.empty(M, topk, dtype=torch.int32, device=gating_output.device)
    rt.require_gpu(gating_output)
    if gating_output.numel() == 0:
        return topk_weights, topk_ids
    # one launch: the kernel reads f16 / bf16 / f32 logits as they are and divides by the row sum
    # itself (the reference's caller does both in separate PyTorch kernels)
    g = gating_output.contiguous()
    if g.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        g = g.float()
    with torch.cuda.device(g.device):
        _lib.call("mi355q_topk_softmax", topk_weights.data_ptr(), topk_ids.data_ptr(), None, g.data_ptr(),
                  M, g.shape[1], topk, int(bool(renormalize)), rt.dtype_code(g.dtype), rt.stream_ptr())
    return topk_weights, topk_ids


def silu_mul_quant(out: torch.Tensor, input: torch.Tensor, scaling: torch.Tensor) -> None:
    """vllm_gcu/kernels/_custom_ops.py:397-400."""
    torch.ops._C.silu_mul_static_int8_quant(out, input, scaling)


# fused moe (vllm_gcu/kernels/_custom_ops.py:490-543)
def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                         num_tokens_post_pad) -> None:
    torch.ops._moe_C.moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                                          num_tokens_post_pad)


def sgl_moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                             num_tokens_post_pad) -> None:
    torch.ops._moe_C.sgl_moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids,
                                              experts_ids, num_tokens_post_pad)


def moe_align_block_size_pad(topk_ids, topk_ids_size, num_experts, block_size, sorted_token_ids,
                             experts_ids, num_tokens_post_pad):
    torch.ops._C.moe_align_block_size_pad(topk_ids, topk_ids_size, num_experts, block_size,
                                          sorted_token_ids, experts_ids, num_tokens_post_pad)


# ---------------------------------------------------------------------------
# activation glue (csrc/torch_bindings.cpp:163-175, 291, 714-766, 1083-1153,
# 1404-1410)
# ---------------------------------------------------------------------------
def _rows_last(t: torch.Tensor):
    return t.numel() // t.shape[-1], t.shape[-1]


def _silu_and_mul_common(out, input, size, rows_per_count=1):
    rt.require_gpu(out, input, size)
    if input.numel() == 0:
        return
    x = input.contiguous()
    rows, d2 = _rows_last(x)
    if not out.is_contiguous() or out.shape[-1] * 2 != d2 or out.dtype != x.dtype:
        raise RuntimeError("silu_and_mul: out must be contiguous [..., d] of the input dtype for input [..., 2d]")
    with torch.cuda.device(x.device):
        _lib.call("mi355q_silu_and_mul", out.data_ptr(), x.data_ptr(), rows, d2 // 2, rt.dtype_code(x.dtype),
                  rt.ptr(size), rows_per_count, rt.stream_ptr())


def _silu_and_mul_impl(result, input):
    _silu_and_mul_common(result, input, None)


def _leading_rows_to_flat(t: torch.Tensor, size: torch.Tensor):
    """``size`` counts entries of the leading dimension (tokens); the kernels work on rows flattened
    over every dimension but the last.  -> (count tensor, rows per counted entry): the product is
    taken inside the kernel, so a captured graph whose count tensor is rewritten between replays
    sees the new value."""
    if size.dtype != torch.int32:
        size = size.to(torch.int32)
    lead = t.shape[0]
    inner = (t.numel() // t.shape[-1]) // max(lead, 1)
    return size, max(int(inner), 1)


def _silu_and_mul_pad_impl(out, input, size):
    _silu_and_mul_common(out, input, *_leading_rows_to_flat(input, size))


def _fp8_out_ok(out, shape):
    if out.dtype not in (torch.float8_e4m3fn, torch.uint8) or not out.is_contiguous() or tuple(out.shape) != tuple(shape):
        raise RuntimeError(f"fp8 output must be a contiguous float8_e4m3fn tensor of shape {tuple(shape)}")


def _group_quant_common(out, scale, input, real_size, group_size, fuse, rows_per_count=1):
    rt.require_gpu(out, scale, input, real_size)
    if input.numel() == 0:
        return
    x = input.contiguous()
    rows, kin = _rows_last(x)
    K = kin // 2 if fuse else kin
    _fp8_out_ok(out, x.shape[:-1] + (K,))
    if scale.dtype != torch.float32 or not scale.is_contiguous() or scale.numel() != rows * (K // group_size):
        raise RuntimeError("per-token-group quant: scale must be contiguous float32 [..., K / group_size]")
    if real_size is not None and real_size.dtype != torch.int32:
        real_size = real_size.to(torch.int32)
    with torch.cuda.device(x.device):
        _lib.call("mi355q_fp8_group_quant", out.data_ptr(), scale.data_ptr(), x.data_ptr(), rows, K,
                  int(group_size), int(fuse), rt.dtype_code(x.dtype), rt.ptr(real_size), rows_per_count,
                  rt.stream_ptr())


def _dynamic_per_token_group_fp8_quant_impl(out, scale, input, group_size):
    _group_quant_common(out, scale, input, None, group_size, False)


def _dynamic_per_token_group_fp8_quant_with_size_impl(out, scale, input, real_size, group_size):
    cnt, rpc = _leading_rows_to_flat(input, real_size)
    _group_quant_common(out, scale, input, cnt, group_size, False, rpc)


def _silu_mul_per_token_group_quant_impl(out, scale, input, group_size):
    _group_quant_common(out, scale, input, None, group_size, True)


def _silu_mul_per_token_group_quant_with_size_impl(out, scale, input, size, group_size):
    cnt, rpc = _leading_rows_to_flat(input, size)
    _group_quant_common(out, scale, input, cnt, group_size, True, rpc)


def _dynamic_per_token_scaled_fp8_quant_impl(result, input, scale, scale_ub):
    # scale_ub is ignored, as in the reference (dynamic_per_token_scaled_fp8_quant.cpp:32-34)
    rt.require_gpu(result, input, scale)
    if input.numel() == 0:
        return
    x = input.contiguous()
    rows, K = _rows_last(x)
    _fp8_out_ok(result, x.shape)
    with torch.cuda.device(x.device):
        _lib.call("mi355q_fp8_token_quant", result.data_ptr(), scale.data_ptr(), x.data_ptr(), rows, K,
                  rt.dtype_code(x.dtype), 0, rt.stream_ptr())


def _static_fp8_common(out, input, scale, real_rows, fuse, rows_per_count=1):
    rt.require_gpu(out, input, scale, real_rows)
    if input.numel() == 0:
        return
    x = input.contiguous()
    rows, kin = _rows_last(x)
    K = kin // 2 if fuse else kin
    _fp8_out_ok(out, x.shape[:-1] + (K,))
    sc = scale.to(torch.float32).reshape(-1)
    if sc.numel() != 1:
        raise RuntimeError("static fp8 quant takes a single scale")
    with torch.cuda.device(x.device):
        _lib.call("mi355q_fp8_static_quant", out.data_ptr(), x.data_ptr(), sc.data_ptr(), rows, K, int(fuse),
                  rt.dtype_code(x.dtype), rt.ptr(real_rows), rows_per_count, rt.stream_ptr())


def _static_scaled_fp8_quant_impl(result, input, scale):
    _static_fp8_common(result, input, scale, None, 0)


def _silu_mul_static_fp8_quant_impl(out, input, scale, real_num_tokens):
    cnt, rpc = _leading_rows_to_flat(input, real_num_tokens)
    _static_fp8_common(out, input, scale, cnt, 1, rpc)


def _mul_static_fp8_quant_impl(out, input, scale, real_num_tokens):
    cnt, rpc = _leading_rows_to_flat(input, real_num_tokens)
    _static_fp8_common(out, input, scale, cnt, 2, rpc)


def _silu_mul_static_int8_quant_impl(result, input, scale):
    # csrc/src/silu_mul_static_int8_quant.cpp:11-28: a 0-d scale is per tensor,
    # anything else per channel of the gated half
    rt.require_gpu(result, input, scale)
    if input.numel() == 0:
        return
    x = input.contiguous()
    rows, kin = _rows_last(x)
    d = kin // 2
    if result.dtype != torch.int8 or tuple(result.shape) != tuple(x.shape[:-1]) + (d,) or not result.is_contiguous():
        raise RuntimeError(f"silu_mul_static_int8_quant: result must be contiguous int8 {tuple(x.shape[:-1]) + (d,)}")
    sc = scale.to(torch.float32).reshape(-1).contiguous()
    if sc.numel() not in (1, d):
        raise RuntimeError(f"silu_mul_static_int8_quant: scale must have 1 or {d} entries, got {sc.numel()}")
    with torch.cuda.device(x.device):
        _lib.call("mi355q_silu_mul_static_int8_quant", result.data_ptr(), x.data_ptr(), sc.data_ptr(),
                  int(sc.numel() > 1), rows, d, rt.dtype_code(x.dtype), rt.stream_ptr())


def _moe_sum_pad_impl(out, input, size, dim, keepdim):
    rt.require_gpu(out, input, size)
    if input.numel() == 0:
        return
    if input.dim() != 3 or dim != 1 or keepdim:
        raise RuntimeError("moe_sum_pad: expects input [M, topk, K], dim=1, keepdim=False")
    x = input.contiguous()
    M, T, K = x.shape
    if not out.is_contiguous() or tuple(out.shape) != (M, K):
        raise RuntimeError("moe_sum_pad: out must be contiguous [M, K]")
    with torch.cuda.device(x.device):
        _lib.call("mi355q_moe_sum", out.data_ptr(), x.data_ptr(), M, T, K, rt.dtype_code(x.dtype),
                  rt.dtype_code(out.dtype), rt.ptr(None if size is None else size.to(torch.int32)),
                  rt.stream_ptr())


_register("_C", "silu_and_mul", "(Tensor! result, Tensor input) -> ()", _silu_and_mul_impl)
_register("_C", "silu_and_mul_pad", "(Tensor(a!) out, Tensor input, Tensor size) -> ()", _silu_and_mul_pad_impl)
_register("_C", "dynamic_per_token_group_fp8_quant",
          "(Tensor! out, Tensor! scale, Tensor input, int group_size) -> ()",
          _dynamic_per_token_group_fp8_quant_impl)
_register("_C", "dynamic_per_token_group_fp8_quant_with_size",
          "(Tensor! out, Tensor! scale, Tensor input, Tensor real_size, int group_size) -> ()",
          _dynamic_per_token_group_fp8_quant_with_size_impl)
_register("_C", "silu_mul_per_token_group_quant",
          "(Tensor! out, Tensor! scale, Tensor input, int group_size) -> ()", _silu_mul_per_token_group_quant_impl)
_register("_C", "silu_mul_per_token_group_quant_with_size",
          "(Tensor(a!) out, Tensor(a!) scale, Tensor input, Tensor size, int group_size) -> ()",
          _silu_mul_per_token_group_quant_with_size_impl)
_register("_C", "dynamic_per_token_scaled_fp8_quant",
          "(Tensor! result, Tensor input, Tensor! scale, Tensor? scale_ub) -> ()",
          _dynamic_per_token_scaled_fp8_quant_impl)
_register("_C", "static_scaled_fp8_quant", "(Tensor! result, Tensor input, Tensor scale) -> ()",
          _static_scaled_fp8_quant_impl)
_register("_C", "mul_static_fp8_quant",
          "(Tensor(a!) out, Tensor input, Tensor scale, Tensor real_num_tokens) -> ()", _mul_static_fp8_quant_impl)
_register("_C", "silu_mul_static_int8_quant", "(Tensor(a!) result, Tensor input, Tensor scale) -> ()",
          _silu_mul_static_int8_quant_impl)
_register("_C", "silu_mul_static_fp8_quant",
          "(Tensor(a!) out, Tensor input, Tensor scale, Tensor real_num_tokens) -> ()",
          _silu_mul_static_fp8_quant_impl)
_register("_moe_C", "moe_sum_pad", "(Tensor(a!) out, Tensor input, Tensor size, int dim, bool keepdim) -> ()",
          _moe_sum_pad_impl)


# ---------------------------------------------------------------------------
# RMS norm and its fusions with the activation quantisers
# (csrc/torch_bindings.cpp:254-317, 852-871, 1124-1143; the fused operators are
# what vllm_gcu/compilation/fusion.py:104-127 substitutes for norm -> quantiser)
# ---------------------------------------------------------------------------
def _rms_common(out, out_scales, input, residual, weight, scale, epsilon, quant_mode, group_size=0):
    rt.require_gpu(out, out_scales, input, residual, weight, scale)
    if input.numel() == 0:
        return
    if input.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"rms_norm: input must be f16/bf16, got {input.dtype}")
    if not input.is_contiguous() or not out.is_contiguous():
        raise RuntimeError("rms_norm: input and output must be contiguous")
    rows, K = _rows_last(input)
    if weight.numel() != K:
        raise RuntimeError(f"rms_norm: weight has {weight.numel()} elements for rows of {K}")
    if tuple(out.shape) != tuple(input.shape):
        raise RuntimeError(f"rms_norm: output shape {tuple(out.shape)} != input shape {tuple(input.shape)}")
    want = {0: input.dtype, 1: torch.float8_e4m3fn, 2: torch.float8_e4m3fn, 3: torch.int8}[quant_mode]
    if out.dtype != want:
        raise RuntimeError(f"rms_norm: output must be {want}, got {out.dtype}")
    if residual is not None and (residual.dtype != input.dtype or tuple(residual.shape) != tuple(input.shape)
                                 or not residual.is_contiguous()):
        raise RuntimeError("rms_norm: residual must match the input (dtype, shape, contiguous)")
    w = weight.to(input.dtype).contiguous()
    sc = None
    if quant_mode in (1, 3):
        sc = scale.to(torch.float32).reshape(-1)
        if sc.numel() != 1:
            raise RuntimeError("rms_norm + static quant takes a single scale")
    if quant_mode == 2:
        if out_scales.dtype != torch.float32 or not out_scales.is_contiguous() or \
                out_scales.numel() != rows * (K // group_size):
            raise RuntimeError("rms_norm + group quant: scales must be contiguous f32 [.., K / group_size]")
    with torch.cuda.device(input.device):
        _lib.call("mi355q_rms_norm", out.data_ptr(), rt.ptr(out_scales), input.data_ptr(), rt.ptr(residual),
                  w.data_ptr(), rt.ptr(sc), float(epsilon), rows, K, quant_mode, int(group_size),
                  rt.dtype_code(input.dtype), rt.stream_ptr())


def _rms_norm_impl(result, input, weight, epsilon):
    _rms_common(result, None, input, None, weight, None, epsilon, 0)


def _fused_add_rms_norm_impl(input, residual, weight, epsilon):
    _rms_common(input, None, input, residual, weight, None, epsilon, 0)


def _rms_norm_static_fp8_quant_impl(result, input, weight, scale, epsilon):
    _rms_common(result, None, input, None, weight, scale, epsilon, 1)


def _fused_add_rms_norm_static_fp8_quant_impl(result, input, residual, weight, scale, epsilon):
    _rms_common(result, None, input, residual, weight, scale, epsilon, 1)


def _rms_norm_per_token_group_quant_fp8_impl(out, scale, input, weight, epsilon, group_size):
    _rms_common(out, scale, input, None, weight, None, epsilon, 2, group_size)


def _fused_add_rms_norm_per_token_group_quant_fp8_impl(out, residual, scale, input, weight, epsilon, group_size):
    _rms_common(out, scale, input, residual, weight, None, epsilon, 2, group_size)


def _rms_norm_static_int8_quant_impl(result, input, weight, scale, epsilon):
    _rms_common(result, None, input, None, weight, scale, epsilon, 3)


def _fused_add_rms_norm_static_int8_quant_impl(result, input, residual, weight, epsilon, scale):
    _rms_common(result, None, input, residual, weight, scale, epsilon, 3)


_register("_C", "rms_norm", "(Tensor! result, Tensor input, Tensor weight, float epsilon) -> ()", _rms_norm_impl)
_register("_C", "fused_add_rms_norm", "(Tensor! input, Tensor! residual, Tensor weight, float epsilon) -> ()",
          _fused_add_rms_norm_impl)
_register("_C", "rms_norm_static_fp8_quant",
          "(Tensor! result, Tensor input, Tensor weight, Tensor scale, float epsilon) -> ()",
          _rms_norm_static_fp8_quant_impl)
_register("_C", "fused_add_rms_norm_static_fp8_quant",
          "(Tensor! result, Tensor input, Tensor! residual, Tensor weight, Tensor scale, float epsilon) -> ()",
          _fused_add_rms_norm_static_fp8_quant_impl)
_register("_C", "rms_norm_per_token_group_quant_fp8",
          "(Tensor! out, Tensor! scale, Tensor input, Tensor weight, float epsilon, int group_size) -> ()",
          _rms_norm_per_token_group_quant_fp8_impl)
_register("_C", "fused_add_rms_norm_per_token_group_quant_fp8",
          "(Tensor! out, Tensor! residual, Tensor! scale, Tensor input, Tensor weight, float epsilon, "
          "int group_size) -> ()", _fused_add_rms_norm_per_token_group_quant_fp8_impl)
_register("_C", "rms_norm_static_int8_quant",
          "(Tensor(a!) result, Tensor input, Tensor weight, Tensor scale, float epsilon) -> ()",
          _rms_norm_static_int8_quant_impl)
_register("_C", "fused_add_rms_norm_static_int8_quant",
          "(Tensor(a!) result, Tensor input, Tensor(a!) residual, Tensor weight, float epsilon, Tensor scale) -> ()",
          _fused_add_rms_norm_static_int8_quant_impl)


# 8bit (vllm_gcu/kernels/_custom_ops.py:298-317)
def scaled_fp8_quant(input: torch.Tensor, scale: Optional[torch.Tensor] = None,
                     num_token_padding: Optional[int] = None, scale_ub: Optional[torch.Tensor] = None,
                     use_per_token_if_dynamic: bool = False,
                     output: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    if scale is None:
        if use_per_token_if_dynamic:
            output = torch.empty_like(input, dtype=torch.float8_e4m3fn)
            shape = input.shape[:-1] + (1,)
            scale = torch.empty(shape, device=input.device, dtype=torch.float32)
            torch.ops._C.dynamic_per_token_scaled_fp8_quant(output, input, scale, scale_ub)
        else:
            raise NotImplementedError("dynamic_scaled_fp8_quant is not implemented for per tensor!")
    else:
        if output is None:
            output = torch.empty_like(input, dtype=torch.float8_e4m3fn)
        torch.ops._C.static_scaled_fp8_quant(output, input, scale)
    return output, scale


# vllm_gcu/kernels/_custom_ops.py:465-486
def per_token_group_quant_fp8(x: torch.Tensor, group_size: int, eps: float = 1e-10,
                              dtype: Optional[torch.dtype] = None, column_major_scales: bool = False,
                              real_token_num: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    dtype = torch.float8_e4m3fn if dtype is None else dtype
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    shape = x.shape[:-1] + (x.shape[-1] // group_size,)
    x_s = torch.empty(shape, device=x.device, dtype=torch.float32)
    if real_token_num is None:
        torch.ops._C.dynamic_per_token_group_fp8_quant(x_q, x_s, x, group_size)
    else:
        torch.ops._C.dynamic_per_token_group_fp8_quant_with_size(x_q, x_s, x, real_token_num, group_size)
    return x_q, x_s


# ---------------------------------------------------------------------------
# fused-MoE grouped GEMM, block-fp8 and weight-only dense GEMMs
# (csrc/torch_bindings.cpp:790-849, 1021-1027)
# ---------------------------------------------------------------------------
_AUTO_KSLAB = os.environ.get("MI355Q_AUTO_KSLAB", "1") != "0"


def _kcontig_weight(w: torch.Tensor):
    """-> (weight tensor, layout code).  K-contiguous weights stream about a
    third faster in the kslab order; a row-major tensor that qualifies is
    converted on first use and the copy cached on it (twice the memory -- the
    method classes convert in place at load time instead; MI355Q_AUTO_KSLAB=0
    turns the implicit conversion off)."""
    from .quantization import rearrange
    if rearrange.is_kslab(w):
        return w, 1
    w = w.contiguous()
    if _AUTO_KSLAB and rearrange.kslab_eligible(w):
        return _converted(w, rearrange.to_kslab), 1
    return w, 0


def _moe_gemm(C, A, B, A_scale, B_scale, gs, B_zp, topk_weights, topk_ids, sorted_token_ids, experts_ids,
              num_tokens_post_pad, mul_routed_weight, topk, block_size, bias, real_token_num):
    """``C.view(-1, N)[t] = A[t // topk] @ W[e(t)]^T (* topk_weights.flat[t])``
    for every id ``t < numel`` listed in ``sorted_token_ids``.  The mode is read
    off the arguments exactly as the reference's wrapper does
    (fused_moe_quant_kernel.cpp:68-76, fused_moe.py:146-172)."""
    rt.require_gpu(C, A, B, A_scale, B_scale, B_zp, topk_weights, topk_ids, sorted_token_ids, experts_ids,
                   num_tokens_post_pad)
    if bias is not None:
        raise RuntimeError("fused_moe kernels take no bias (fused_moe_quant_kernel.cpp:77)")
    numel = topk_ids.numel()
    if numel == 0 or A.numel() == 0:
        return
    A = A.contiguous()
    K = A.shape[-1]
    N = C.shape[-1]
    if not C.is_contiguous():
        raise RuntimeError("fused_moe: C must be contiguous")
    zk, zp, group = _lib.ZP_NONE, None, int(gs)
    a_scale = w_scale = None
    if A_scale is not None and A.dtype in (torch.float16, torch.bfloat16) and B.dtype == torch.int8 \
            and A_scale.dim() == 2 and A_scale.shape[-1] == K and A_scale.dtype == A.dtype:
        # static int8 experts (w8a8.py:174-342): 16-bit activations plus per-expert, per-channel reciprocal
        # input scales [E, K].  Each (token, slot) row is quantised with its expert's vector, then the
        # int8 grouped GEMM reads one row per slot.
        rec = A_scale.contiguous()
        # rows of pads and of non-local experts are never read by the GEMM (zeros, so that nothing is undefined)
        Aq = torch.zeros((numel, K), dtype=torch.int8, device=A.device)
        with torch.cuda.device(A.device):
            _lib.call("mi355q_moe_expert_int8_quant", Aq.data_ptr(), A.data_ptr(), rec.data_ptr(),
                      sorted_token_ids.data_ptr(), experts_ids.data_ptr(), num_tokens_post_pad.data_ptr(),
                      sorted_token_ids.numel(), int(block_size), numel, int(topk), rec.shape[0], K,
                      rt.dtype_code(A.dtype), rt.stream_ptr())
        A, A_scale, topk = Aq, None, 1
        mode = _lib.Q_INT8
        w_scale = B_scale.to(torch.float32).reshape(B.shape[0], -1).contiguous()
        w = B.contiguous()
        act_code = _lib.F16
    elif A_scale is not None:
        if A.dtype == torch.float8_e4m3fn:
            mode = _lib.Q_FP8_BLOCK
            a_scale = A_scale.to(torch.float32).contiguous()
            w_scale = B_scale.to(torch.float32).contiguous()
            w = B.contiguous()
            if w.shape[-1] != K:
                raise RuntimeError(f"fp8 expert weights must be [E, N, K]; got {tuple(w.shape)} for K={K}")
        elif A.dtype == torch.int8:
            mode = _lib.Q_INT8
            a_scale = A_scale.to(torch.float32).reshape(-1)
            if a_scale.numel() == 1:                    # one static scale for every token
                a_scale = a_scale.expand(A.shape[0])
            a_scale = a_scale.contiguous()
            if a_scale.numel() != A.shape[0]:
                raise RuntimeError("int8 MoE needs one activation scale, or one per token")
            w_scale = B_scale.to(torch.float32).reshape(B.shape[0], -1).contiguous()
            w = B.contiguous()
        else:
            raise RuntimeError(f"A_scale given but activations are {A.dtype}")
        act_code = _lib.F16
    elif B.dtype == torch.int32 or (B.dtype in (torch.uint8, torch.int8) and B.shape[-1] * 2 == K):
        mode = _lib.Q_W4A16
        w = _slab_weight(B, transposed=True)
        if w.shape[-2] * 8 != K or w.shape[-1] != N:
            raise RuntimeError(f"fused_moe: int4 experts of shape {tuple(w.shape)} do not fit K={K}, N={N}")
        zp, zk = _zero_points(B_zp, A.dtype, B_scale)
        w_scale = B_scale.contiguous()
        if w_scale.dtype != A.dtype:
            w_scale = w_scale.to(A.dtype)
        if zp is not None:
            zp = zp.contiguous()
        if group <= 0:
            group = K
        ne, groups = w.shape[0], K // group
        if w_scale.numel() != ne * groups * N:
            raise RuntimeError(f"fused_moe: int4 expert scales of shape {tuple(w_scale.shape)} do not fit "
                               f"{ne} experts x {groups} groups x {N} columns")
        if zp is not None and zp.numel() != ne * groups * (N // 8 if zk == _lib.ZP_PACKED else N):
            raise RuntimeError(f"fused_moe: int4 expert zero-points of shape {tuple(zp.shape)} do not fit "
                               f"{ne} experts x {groups} groups x {N} columns")
        act_code = rt.dtype_code(A.dtype)
    elif B.dtype == torch.int8:
        mode = _lib.Q_W8A16
        w = B.contiguous()
        if group in (64, 128) and B_scale.dim() == 3 and B_scale.shape[1] == K // group:
            w_scale = B_scale.to(A.dtype).contiguous()                    # [E, K/g, N]
        else:
            w_scale = B_scale.reshape(B.shape[0], -1).to(A.dtype).contiguous()
            if w_scale.shape[1] != N:
                raise RuntimeError(f"w8a16 experts: scales {tuple(B_scale.shape)} fit neither [E, N] nor [E, K/g, N]")
            group = -1
        act_code = rt.dtype_code(A.dtype)
    elif B.dtype == A.dtype and B_scale is None:
        mode = _lib.Q_NONE
        w = B.contiguous()
        act_code = rt.dtype_code(A.dtype)
    else:
        raise RuntimeError(f"fused_moe: cannot infer the quantisation mode from A {A.dtype} / B {B.dtype}")
    layout = 0
    if mode != _lib.Q_W4A16:
        w, layout = _kcontig_weight(w)
    E = w.shape[0]
    tw = None
    if mul_routed_weight:
        tw = topk_weights.to(torch.float32).contiguous()
        if tw.numel() != numel:
            raise RuntimeError("fused_moe: topk_weights must have one entry per (token, slot)")
    for t in (sorted_token_ids, experts_ids, num_tokens_post_pad):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("fused_moe: sorted_token_ids / experts_ids / num_tokens_post_pad must be contiguous int32")
    if sorted_token_ids.numel() < experts_ids.numel() * block_size:
        raise RuntimeError("fused_moe: sorted_token_ids is shorter than experts_ids * block_size")
    with torch.cuda.device(A.device):
        ws_ptr = ws_bytes = 0
        need = _lib.load().mi355q_moe_gemm_workspace_bytes(mode, numel, int(block_size), experts_ids.numel(), E, K, N)
        if need:
            # behind the first MiB of the shared scratch, which holds arrival counters that stay zero
            ws = rt.workspace(A.device, need + _WS_COUNTER_BYTES)
            ws_ptr, ws_bytes = ws.data_ptr() + _WS_COUNTER_BYTES, ws.numel() - _WS_COUNTER_BYTES
        _lib.call("mi355q_moe_gemm", C.data_ptr(), A.data_ptr(), w.data_ptr(), rt.ptr(a_scale), rt.ptr(w_scale),
                  rt.ptr(zp), zk, mode, group, rt.ptr(tw), sorted_token_ids.data_ptr(), experts_ids.data_ptr(),
                  num_tokens_post_pad.data_ptr(), numel, int(topk), int(block_size), experts_ids.numel(), E, K, N,
                  act_code, rt.dtype_code(C.dtype), layout, ws_ptr, ws_bytes, rt.stream_ptr())


def _fused_moe_quant_kernel_impl(C, A, B, A_scale, B_scale, gs, B_zp, topk_weights, topk_ids, sorted_token_ids,
                                 experts_ids, num_tokens_post_pad, mul_routed_weight, topk, block_size, bias,
                                 real_token_num):
    _moe_gemm(C, A, B, A_scale, B_scale, gs, B_zp, topk_weights, topk_ids, sorted_token_ids, experts_ids,
              num_tokens_post_pad, mul_routed_weight, topk, block_size, bias, real_token_num)


def _fused_moe_quant_kernel_ex_impl(C, A, B, A_scale, B_scale, B_zero, bias, topk_weights, topk_ids,
                                    sorted_token_ids, experts_ids, num_tokens_post_pad, real_token_num,
                                    mul_routed_weight, topk, block_size, group_k, group_n):
    """w4a8-fp8 experts (fused_moe_quant_kernel_ex.cpp:13-45, called from
    fused_moe.py:173-195): fp8 activations with one static scale, symmetric int4
    weights with fp32 group scales ``[E, K/group_k, N]``.

    ``A_scale`` is what the reference passes there: the *reciprocal* of the
    scale the activations were quantised with (``layer.w13_input_scale_rec``,
    w4a8.py:222-235).  The vendor kernel's arithmetic is not part of the
    reference; with ``static_scaled_fp8_quant`` dividing by its scale, the only
    reading under which quantise -> GEMM reproduces the float layer is
    ``C = (A @ dequant(B)) / A_scale``, which is what runs here.  fp8 values
    are widened exactly to C's dtype and multiplied on the fp16/bf16 matrix
    pipe with fp32 accumulation."""
    rt.require_gpu(C, A, B, A_scale, B_scale, topk_weights, topk_ids, sorted_token_ids, experts_ids,
                   num_tokens_post_pad)
    if bias is not None:
        raise RuntimeError("fused_moe_quant_kernel_ex takes no bias")
    if B_zero is not None and B_zero.numel():
        raise RuntimeError("fused_moe_quant_kernel_ex: w4a8 experts are symmetric (w4a8.py:143 passes no zeros)")
    if group_n not in (-1, 1):
        raise RuntimeError(f"fused_moe_quant_kernel_ex: group_n={group_n}: scales are per output channel")
    numel = topk_ids.numel()
    if numel == 0 or A.numel() == 0:
        return
    if A.dtype != torch.float8_e4m3fn:
        raise RuntimeError(f"fused_moe_quant_kernel_ex: activations must be float8_e4m3fn, got {A.dtype}")
    if not C.is_contiguous() or C.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("fused_moe_quant_kernel_ex: C must be contiguous f16/bf16")
    A = A.contiguous()
    K, N = A.shape[-1], C.shape[-1]
    if B.dtype == torch.int32:
        w = B                                           # slab tensor from this build's loader
    elif B.dtype in (torch.int8, torch.uint8) and B.shape[-1] * 2 == K:
        w = _converted(B, rearrange.from_reference_w4a8)
    else:
        raise RuntimeError(f"fused_moe_quant_kernel_ex: int4 experts expected, got {B.dtype} {tuple(B.shape)}")
    if w.shape[-2] * 8 != K or w.shape[-1] != N:
        raise RuntimeError(f"fused_moe_quant_kernel_ex: weights {tuple(w.shape)} do not match K={K}, N={N}")
    E = w.shape[0]
    w_scale = B_scale.to(torch.float32).contiguous()
    if tuple(w_scale.shape) != (E, K // group_k, N):
        raise RuntimeError(f"fused_moe_quant_kernel_ex: scales {tuple(w_scale.shape)} != {(E, K // group_k, N)}")
    out_scale = _converted(A_scale, lambda t: (1.0 / t.detach().to(torch.float32)).reshape(-1)[:1].contiguous())
    a16 = torch.empty(A.shape, dtype=C.dtype, device=A.device)
    tw = None
    if mul_routed_weight:
        tw = topk_weights.to(torch.float32).contiguous()
        if tw.numel() != numel:
            raise RuntimeError("fused_moe: topk_weights must have one entry per (token, slot)")
    for t in (sorted_token_ids, experts_ids, num_tokens_post_pad):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("fused_moe: sorted_token_ids / experts_ids / num_tokens_post_pad must be contiguous int32")
    if sorted_token_ids.numel() < experts_ids.numel() * block_size:
        raise RuntimeError("fused_moe: sorted_token_ids is shorter than experts_ids * block_size")
    code = rt.dtype_code(C.dtype)
    with torch.cuda.device(A.device):
        _lib.call("mi355q_fp8_to_half", a16.data_ptr(), A.data_ptr(), A.numel(), code, rt.stream_ptr())
        _lib.call("mi355q_moe_gemm", C.data_ptr(), a16.data_ptr(), w.data_ptr(), out_scale.data_ptr(),
                  w_scale.data_ptr(), 0, _lib.ZP_NONE, _lib.Q_W4_F32SCALE, int(group_k), rt.ptr(tw),
                  sorted_token_ids.data_ptr(), experts_ids.data_ptr(), num_tokens_post_pad.data_ptr(), numel,
                  int(topk), int(block_size), experts_ids.numel(), E, K, N, code, code, 0, 0, 0, rt.stream_ptr())


def _fused_moe_kernel_impl(C, A, B, topk_weights, topk_ids, sorted_topk_ids, expert_ids, num_tokens_post_pad,
                           mul_routed_weight, topk, block_size, bias):
    _moe_gemm(C, A, B, None, None, 0, None, topk_weights, topk_ids, sorted_topk_ids, expert_ids,
              num_tokens_post_pad, mul_routed_weight, topk, block_size, bias, None)


def _kcontig(out, a, w, a_scale, w_scale, bias, mode, group):
    rt.require_gpu(out, a, w, a_scale, w_scale, bias)
    a2 = a.reshape(-1, a.shape[-1]).contiguous()
    M, K = a2.shape
    N = w.shape[0]
    if w.shape[1] != K or not w.is_contiguous():
        raise RuntimeError(f"weight must be contiguous [N, K]; got {tuple(w.shape)} for K={K}")
    if not out.is_contiguous() or out.shape[-1] != N or out.numel() != M * N:
        raise RuntimeError("output must be contiguous [.., N]")
    if bias is not None:
        bias = bias.to(out.dtype).contiguous()
    act = _lib.F16 if a.dtype in (torch.float8_e4m3fn, torch.int8) else rt.dtype_code(a.dtype)
    w, layout = _kcontig_weight(w)
    with torch.cuda.device(a.device):
        _lib.call("mi355q_kcontig_gemm", out.data_ptr(), a2.data_ptr(), w.data_ptr(), rt.ptr(a_scale),
                  rt.ptr(w_scale), rt.ptr(bias), mode, group, M, K, N, act, rt.dtype_code(out.dtype),
                  layout, rt.stream_ptr())


# the MFMA tile kernel beats the weight-streaming kernel above 64 rows once its tiles fill a good part of
# the chip (measured, K 8192 N 28672 = 224 tiles: M 65..128 69..73 us against 87..119 us, M 64 68 us
# against 73 us for the streamer's last single-block size; K 7168 N 4096 = 32 tiles: 52 us against
# 37..53 us at M 65..128, so few tiles stay with the streamer).  The tile kernel needs about 1 us
# per K block however few tiles there are; the streamer's time grows with the rows: they cross at
# 48..64 tiles (K 7168 N 4096: 32 tiles 56 against 31 us, 64 tiles 55 against 58 us, 96 tiles 56
# against 85 us; the same on K 4096 N 4096, K 2048 N 7168 and K 7168 N 2048)
_FP8_TILE_MIN_M = 64
_FP8_STAGE_SCALES = True      # room in the workspace for the activation scales in K block major order (tile kernel)
_FP8_TILE_MIN_TILES = 64


def _linear_quant_impl(out, lhs, rhs, bias, lhs_scale, rhs_scale):
    """fp8 block-scaled GEMM (linear_quant.cpp:16-95): lhs fp8 [.., K] with
    scales [.., K/128]; rhs fp8 [N, K] with scales [N/128, K/128]."""
    if lhs.numel() == 0:
        return
    if lhs.dtype != torch.float8_e4m3fn or rhs.dtype != torch.float8_e4m3fn:
        raise RuntimeError("linear_quant: operands must be float8_e4m3fn")
    M, N, K = lhs.numel() // lhs.shape[-1], rhs.shape[0], lhs.shape[-1]
    tiles = -(-M // 256) * (N // 128)               # 256 x 128 output tiles, one workgroup each
    # (from 33 rows on a layer of 128 tiles or more: the tile kernel's wavefronts without rows only copy,
    # K 8192 x N 28672 at M = 40 / 48 / 64: 59.0 / 62.3 / 68.7 -> 55.5 / 56.3 / 53.6 us; 112 tiles: the streamer stays ahead)
    # (and, whatever the tile count, where the library plans K ranges side by side that fill the chip:
    # from 65 rows, and from 25 / 33 rows on where K is long, see fp8_split_min_rows)
    need = _lib.load().mi355q_fp8_gemm_workspace_bytes(M, N, K) \
        if M > _FP8_TILE_MIN_M // 4 and N % 128 == 0 and K % 128 == 0 else 0
    if (need or (M > _FP8_TILE_MIN_M and tiles >= _FP8_TILE_MIN_TILES)
            or (M > _FP8_TILE_MIN_M // 2 and tiles >= 2 * _FP8_TILE_MIN_TILES)) \
            and N % 128 == 0 and K % 128 == 0 \
            and out.dtype in (torch.float16, torch.bfloat16) \
            and rhs.dim() == 2 and rhs.is_contiguous() and out.is_contiguous():
        # prefill-sized M: the MFMA tile kernel (the weight-streaming kernel re-reads the weights per 64 rows)
        rt.require_gpu(out, lhs, rhs, bias, lhs_scale, rhs_scale)
        from .quantization import rearrange
        a2 = lhs.reshape(M, K).contiguous()
        xs = lhs_scale.to(torch.float32).reshape(M, -1).contiguous()
        ws = rhs_scale.to(torch.float32).contiguous()
        if tuple(xs.shape) != (M, K // 128) or tuple(ws.shape) != (N // 128, K // 128):
            raise RuntimeError(f"linear_quant: scales {tuple(xs.shape)} / {tuple(ws.shape)} do not match "
                               f"M={M} N={N} K={K} with 128 x 128 blocks")
        b = None if bias is None else bias.to(out.dtype).contiguous()
        with torch.cuda.device(lhs.device):
            # behind the partial sums of a K split (or the first MiB): room for the activation scales in K block major order
            stage = (M + 15) // 16 * 16 * (K // 128) * 4 if _FP8_STAGE_SCALES else 0
            total = (need or ((1 << 20) if stage else 0)) + stage
            wsp = rt.workspace(lhs.device, total) if total else None
            _lib.call("mi355q_fp8_block_gemm_ws", out.data_ptr(), a2.data_ptr(), rhs.data_ptr(), xs.data_ptr(),
                      ws.data_ptr(), rt.ptr(b), M, N, K, K, 0 if rearrange.is_kslab(rhs) else K, N,
                      rt.dtype_code(out.dtype), rt.ptr(wsp), 0 if wsp is None else wsp.numel(), rt.stream_ptr())
        return
    _kcontig(out, lhs, rhs, lhs_scale.to(torch.float32).reshape(-1, lhs_scale.shape[-1]).contiguous(),
             rhs_scale.to(torch.float32).contiguous(), bias, _lib.Q_FP8_BLOCK, 128)


def _weight_only_quant_impl(output, input, qweight, bias, scale, group_size):
    """W8A16 (weight_only_quant.cpp:28-101): qweight int8 [N, K]; scale [N] per
    channel (group_size -1) or [K/g, N] for groups of 64 / 128 along K, the
    shapes GPTQGCULinearMethod leaves behind for 8-bit checkpoints (gptq.py:262-270)."""
    if input.numel() == 0:
        return
    if qweight.dtype != torch.int8:
        raise RuntimeError("weight_only_quant: qweight must be int8 [N, K]")
    N, K = qweight.shape
    if scale.numel() == N:
        _kcontig(output, input, qweight, None, scale.reshape(-1).to(input.dtype).contiguous(), bias, _lib.Q_W8A16, -1)
        return
    g = int(group_size)
    if g not in (64, 128) or tuple(scale.shape) != (K // g, N):
        raise RuntimeError(f"weight_only_quant: scales {tuple(scale.shape)} with group_size {group_size}: expected "
                           f"[N] or [K/g, N] with g = 64 or 128")
    _kcontig(output, input, qweight, None, scale.to(input.dtype).contiguous(), bias, _lib.Q_W8A16, g)


# the three operators below are registered from C++ function pointers in the
# reference (torch_bindings.cpp:793-817), so callers pass everything by position
_register("_C", "fused_moe_quant_kernel",
          "(Tensor(a!) C, Tensor A, Tensor B, Tensor? A_scale, Tensor? B_scale, int gs, Tensor? B_zp, "
          "Tensor topk_weights, Tensor topk_ids, Tensor sorted_token_ids, Tensor experts_ids, "
          "Tensor num_tokens_post_pad, bool mul_routed_weight, int topk, int block_size, Tensor? bias, "
          "Tensor? real_token_num) -> ()", _fused_moe_quant_kernel_impl)
_register("_C", "fused_moe_quant_kernel_ex",
          "(Tensor(a!) C, Tensor A, Tensor B, Tensor A_scale, Tensor B_scale, Tensor? B_zero, Tensor? bias, "
          "Tensor topk_weights, Tensor topk_ids, Tensor sorted_token_ids, Tensor experts_ids, "
          "Tensor num_tokens_post_pad, Tensor? real_token_num, bool mul_routed_weight, int topk, "
          "int block_size, int group_k, int group_n) -> ()", _fused_moe_quant_kernel_ex_impl)
_register("_C", "fused_moe_kernel",
          "(Tensor(a!) C, Tensor A, Tensor B, Tensor topk_weights, Tensor topk_ids, Tensor sorted_topk_ids, "
          "Tensor expert_ids, Tensor num_tokens_post_pad, bool mul_routed_weight, int topk, int block_size, "
          "Tensor? bias) -> ()", _fused_moe_kernel_impl)
_register("_C", "linear_quant",
          "(Tensor! out, Tensor lhs, Tensor rhs, Tensor? bias, Tensor lhs_scale, Tensor rhs_scale) -> ()",
          _linear_quant_impl)
_register("_C", "weight_only_quant",
          "(Tensor! output, Tensor input, Tensor qweight, Tensor? bias, Tensor scale, int group_size) -> ()",
          _weight_only_quant_impl)


# ---------------------------------------------------------------------------
# fused q / kv projections (csrc/src/fused_qkv_proj.cpp:14-23,
# fused_qkv_gemm_quant.cpp:12-20; defs torch_bindings.cpp:1204-1217)
# ---------------------------------------------------------------------------
# The reference forwards both straight to its vendor library and has neither a
# Python caller nor a test nor a description of them, so their arithmetic is
# unpinned.  They are built as what the signatures say: one quantised GEMM over
# the merged weight whose output columns are split into ``q`` (the first
# q.shape[-1]) and ``kv`` (the rest) -- the merged q_a / kv_a projection of an
# MLA layer.
def _split_qkv(q, kv, merged):
    nq, nkv = q.shape[-1], kv.shape[-1]
    if merged.shape[-1] != nq + nkv:
        raise RuntimeError(f"fused qkv: weight has {merged.shape[-1]} output columns, q + kv need {nq} + {nkv}")
    q.copy_(merged[:, :nq].reshape(q.shape))
    kv.copy_(merged[:, nq:].reshape(kv.shape))


def _fused_qkv_proj_impl(q, kv, x, weight, x_scale, weight_scale, group_size):
    """fp8 block-scaled: x fp8 [.., K] with scales [.., K/128], weight fp8 [Nq + Nkv, K] with scales
    [(Nq + Nkv)/128, K/128]; the arithmetic of linear_quant."""
    rt.require_gpu(q, kv, x, weight, x_scale, weight_scale)
    if x.numel() == 0:
        return
    if int(group_size) != 128:
        raise RuntimeError(f"fused_qkv_proj: group_size {group_size}: the fp8 block size is 128")
    x2 = x.reshape(-1, x.shape[-1])
    merged = torch.empty((x2.shape[0], weight.shape[0]), dtype=q.dtype, device=q.device)
    _linear_quant_impl(merged, x2, weight, None, x_scale, weight_scale)
    _split_qkv(q, kv, merged)


def _fused_qkv_gemm_quant_impl(q, kv, x, weight, scale, zeros, group_size):
    """W4A16: the operands of gptq_gemm_gcu (int4 weight in the slab or any reference layout,
    group scales, zeros in any of the accepted forms)."""
    rt.require_gpu(q, kv, x, weight, scale, zeros)
    if x.numel() == 0:
        return
    merged = w4a16_gemm(x.reshape(-1, x.shape[-1]), weight, scale, zeros if zeros.numel() else None, None,
                        int(group_size))
    _split_qkv(q, kv, merged.to(q.dtype))


_register("_C", "fused_qkv_proj",
          "(Tensor(a!) q, Tensor(a!) kv, Tensor x, Tensor weight, Tensor x_scale, Tensor weight_scale, "
          "int group_size) -> ()", _fused_qkv_proj_impl)
_register("_C", "fused_qkv_gemm_quant",
          "(Tensor(a!) q, Tensor(a!) kv, Tensor x, Tensor weight, Tensor scale, Tensor zeros, "
          "int group_size) -> ()", _fused_qkv_gemm_quant_impl)


# vllm_gcu/kernels/_custom_ops.py:564-579
def w8a8_block_fp8_matmul(A: torch.Tensor, B: torch.Tensor, As: torch.Tensor, Bs: torch.Tensor,
                          block_size: List[int], output_dtype: torch.dtype = torch.float16,
                          bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    N, _ = B.shape
    C_shape = A.shape[:-1] + (N,)
    C = A.new_empty(C_shape, dtype=output_dtype)
    torch.ops._C.linear_quant(C, A, B, bias, As, Bs)
    return C
