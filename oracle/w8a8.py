"""W8A8 int8 path on the CPU (numpy / CPU torch).  Test infrastructure only.

* per-token dynamic int8 quantisation
  (csrc/src/dynamic_scaled_int8_quant.cpp:12-19; the arithmetic is upstream
  vLLM's: ``scale = absmax / 127``, ``q = sat_s8(rne(x * (127 / absmax)))``),
* static int8 quantisation (csrc/src/static_scaled_int8_quant.cpp:12-28:
  the reciprocal of the scale is taken and rounded to the *input* dtype, then
  ``q = sat_s8(rne(x * inv))``),
* exact int32 GEMM and the scaled epilogue of ``cutlass_scaled_mm`` /
  ``dot_bias_quant`` (csrc/src/cutlass_scaled_mm.cpp:12-36,
  csrc/src/dot_bias_quant.cpp:12-24).
"""
import numpy as np
import torch


def dynamic_scaled_int8_quant(x: np.ndarray):
    """x float [M, K] -> (q int8 [M, K], scales float32 [M, 1]).

    All arithmetic in float32.  A row of zeros has scale 0 and quantises to 0
    (upstream: 0 * inf = nan converts to 0).
    """
    xf = x.astype(np.float32)
    absmax = np.max(np.abs(xf), axis=-1, keepdims=True).astype(np.float32)
    scales = (absmax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = (np.float32(127.0) / absmax).astype(np.float32)
        y = (xf * inv).astype(np.float32)
    y = np.where(np.isnan(y), np.float32(0), y)
    q = np.clip(np.rint(y), -128, 127).astype(np.int8)
    return q, scales


def static_scaled_int8_quant(x: np.ndarray, scale: np.ndarray):
    """x float16/float32 [M, K]; scale float32 scalar or [K] -> int8 [M, K].

    The reciprocal is rounded to x's dtype (static_scaled_int8_quant.cpp:21,
    24); the product is evaluated in float32 and rounded half-to-even.
    """
    inv = (np.float32(1.0) / np.asarray(scale, dtype=np.float32)).astype(x.dtype)
    y = x.astype(np.float32) * inv.astype(np.float32)
    return np.clip(np.rint(y), -128, 127).astype(np.int8)


def moe_expert_int8_quant(x: np.ndarray, scale_rec: np.ndarray, topk_ids: np.ndarray) -> np.ndarray:
    """Static per-expert, per-input-channel quantisation of fused-MoE activations: for every
    (token, slot) id t with expert e, ``q[t] = sat_s8(rne(x[t // topk] * scale_rec[e]))``, product in
    float32.  ``scale_rec [E, K]`` holds reciprocals, as the reference's loader stores
    ``w13_in_scales`` / ``w2_in_scales`` (vllm_gcu/kernels/quantization/w8a8.py:226-236, 277-289) and
    hands them, with the un-quantised activations, to its vendor grouped GEMM
    (vllm_gcu/kernels/prepare_finalize.py:62-64, w8a8.py:339-340).  Parity unpinned: the vendor
    kernel's rounding is not in the reference; this is the build's own definition."""
    M, K = x.shape
    flat = topk_ids.reshape(-1)
    topk = topk_ids.shape[-1] if topk_ids.ndim > 1 else 1
    rows = np.arange(flat.size) // topk
    y = x[rows].astype(np.float32) * scale_rec[flat].astype(np.float32)
    return np.clip(np.rint(y), -128, 127).astype(np.int8)


def int8_gemm_i32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Exact ``a[M, K] @ b[K, N]`` in int32 for int8 operands.

    Evaluated as float32 matmuls over K-chunks of 1024: every partial sum is
    an integer below 1024 * 128 * 128 = 2**24, hence exact in float32; the
    chunks are then added in int64.
    """
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    acc = np.zeros((M, N), dtype=np.int64)
    bt = torch.from_numpy(np.ascontiguousarray(b))
    at = torch.from_numpy(np.ascontiguousarray(a))
    for k0 in range(0, K, 1024):
        pa = at[:, k0:k0 + 1024].float()
        pb = bt[k0:k0 + 1024].float()
        acc += torch.matmul(pa, pb).numpy().astype(np.int64)
    assert np.abs(acc).max(initial=0) < 2 ** 31
    return acc.astype(np.int32)


def scaled_mm_epilogue(acc: np.ndarray, x_scale, w_scale, bias=None) -> np.ndarray:
    """float32 ``acc * x_scale[M or 1] * w_scale[N or 1] (+ bias)``.

    x_scale: scalar, [1], [M] or [M, 1]; w_scale: scalar, [1], [N] or [N, 1]
    (cutlass_scaled_mm.cpp:23-32 unsqueezes a 0-d x_scale and squeezes an
    [N, 1] w_scale).  The product is formed as ``(float(acc) * x_scale) *
    w_scale`` in float32; the caller casts to the output dtype.
    """
    xs = np.asarray(x_scale, dtype=np.float32).reshape(-1, 1)
    ws = np.asarray(w_scale, dtype=np.float32).reshape(1, -1)
    out = (acc.astype(np.float32) * xs).astype(np.float32) * ws
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.float32).reshape(1, -1)
    return out.astype(np.float32)


def weight_only_int8(x: np.ndarray, w_nk: np.ndarray, scale: np.ndarray,
                     group_size: int, bias=None) -> np.ndarray:
    """W8A16: ``x @ (w[N, K] * scale).T`` in float32
    (csrc/src/weight_only_quant.cpp:28-101); scale [N] (per channel,
    group_size -1) or [K/g, N]."""
    N, K = w_nk.shape
    wf = w_nk.astype(np.float32)
    if group_size in (-1, 0) or scale.ndim == 1:
        wd = wf * scale.astype(np.float32).reshape(N, 1)
    else:
        g = group_size
        wd = (wf.reshape(N, K // g, g) *
              scale.astype(np.float32).T.reshape(N, K // g, 1)).reshape(N, K)
    out = torch.matmul(torch.from_numpy(x.astype(np.float32)),
                       torch.from_numpy(np.ascontiguousarray(wd.T))).numpy()
    if bias is not None:
        out = out + bias.astype(np.float32)[None, :]
    return out


# ----------------------------------------------------------------------------
# This build's streaming order for K-contiguous weights ("kslab")
# ----------------------------------------------------------------------------
def kslab_pack(w: np.ndarray) -> np.ndarray:
    """[.., N, K] of 1- or 2-byte elements -> same shape/dtype, bytes in the
    order ``[N/64][K/128][4 tiles][2*elem_bytes vectors][64 lanes][16 B]``: lane
    ``l`` of vector ``v`` of tile ``i`` in (row group G, K block kb) holds the 16
    bytes at byte offset ``(128 kb + 32 (l // 16)) * elem_bytes + 16 v`` of row
    ``64 G + 16 i + l % 16``.  No counterpart in the reference (its fp8 / int8
    weights stay row-major, vllm_gcu/kernels/quantization/fp8.py:72-166);
    pinned by :func:`kslab_unpack`, a scalar walk of the same definition."""
    wb = w.dtype.itemsize
    N, K = w.shape[-2:]
    assert wb in (1, 2) and N % 64 == 0 and K % 128 == 0
    lead = w.shape[:-2]
    b = np.ascontiguousarray(w).view(np.uint8).reshape(-1, N // 64, 4, 16, K // 128, 4, 2 * wb, 16)
    #                          axes:  e, G, i, r, kb, q, v, byte  ->  e, G, kb, i, v, q, r, byte
    out = np.ascontiguousarray(b.transpose(0, 1, 4, 2, 6, 5, 3, 7))
    return out.reshape(-1).view(w.dtype).reshape(*lead, N, K)


def kslab_unpack(p: np.ndarray) -> np.ndarray:
    """Inverse of :func:`kslab_pack` for one matrix, as a scalar index walk."""
    wb = p.dtype.itemsize
    N, K = p.shape
    flat = np.ascontiguousarray(p).view(np.uint8).reshape(-1)
    rows = np.zeros((N, K * wb), dtype=np.uint8)
    idx = 0
    for G in range(N // 64):
        for kb in range(K // 128):
            for i in range(4):
                for v in range(2 * wb):
                    for lane in range(64):
                        n = 64 * G + 16 * i + lane % 16
                        off = (128 * kb + 32 * (lane // 16)) * wb + 16 * v
                        rows[n, off:off + 16] = flat[idx:idx + 16]
                        idx += 16
    return rows.reshape(-1).view(p.dtype).reshape(N, K)
