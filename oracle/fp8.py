"""fp8-e4m3fn quantisation and the 128x128 block-scaled GEMM on the CPU.

Test infrastructure only.

* ``per_token_group_quant_fp8`` (vllm_gcu/kernels/_custom_ops.py:465-486 ->
  csrc/src/dynamic_per_token_group_fp8_quant.cpp:15-84): per (token,
  group) ``s = max(absmax, eps) / 448`` and ``q = e4m3fn(clamp(x / s,
  -448, 448))``; 448 is FP8_E4M3_MAX (csrc/src/native_vllm.h:34).
* ``w8a8_block_fp8_matmul`` (_custom_ops.py:564-579 ->
  csrc/src/linear_quant.cpp:16-95): ``C = sum_kb (A[:, kb] @ B[:, kb].T) *
  As[:, kb] * Bs[nb, kb]``.
* ``cutlass_scaled_mm`` on fp8 operands (csrc/src/cutlass_scaled_mm.cpp:12-36,
  reached from the non-block branch of vllm_gcu/kernels/quantization/fp8.py:68-69):
  ``C = (A @ B.T) * a_scale[m] * b_scale[n] (+ bias)``.
"""
import numpy as np
import torch

FP8_MAX = 448.0


def e4m3fn_decode_table() -> np.ndarray:
    """float64 value of each of the 256 e4m3fn codes, from the bit fields:
    sign(1) exponent(4, bias 7) mantissa(3); exponent 0 is subnormal
    (m/8 * 2**-6); 0x7f / 0xff are NaN; there are no infinities."""
    t = np.zeros(256, dtype=np.float64)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 7
        if e == 0xF and m == 7:
            t[code] = np.nan
        elif e == 0:
            t[code] = s * (m / 8.0) * 2.0 ** -6
        else:
            t[code] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return t


def e4m3fn_encode_bruteforce(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even onto the e4m3fn grid by exhaustive search over
    the decode table (inputs must already be within +-448).  Slow; exists to
    pin :func:`to_e4m3fn`."""
    tab = e4m3fn_decode_table()
    pos = [(tab[c], c) for c in range(0x7F)]                 # 0 .. 448
    vals = np.array([p[0] for p in pos])
    out = np.zeros(x.shape, dtype=np.uint8)
    flat = x.astype(np.float64).reshape(-1)
    o = out.reshape(-1)
    for i, v in enumerate(flat):
        a = abs(v)
        d = np.abs(vals - a)
        best = int(np.argmin(d))
        ties = np.nonzero(d == d[best])[0]
        if len(ties) > 1:
            best = int([c for c in ties if c % 2 == 0][0])   # even mantissa lsb
        o[i] = best | (0x80 if (v < 0 or (v == 0 and np.signbit(v))) else 0)
    return out


def to_e4m3fn(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn codes (uint8), round-half-even, input pre-clamped."""
    t = torch.from_numpy(np.ascontiguousarray(x.astype(np.float32)))
    return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def from_e4m3fn(codes: np.ndarray) -> np.ndarray:
    return e4m3fn_decode_table()[codes.astype(np.uint8)].astype(np.float32)


def per_token_group_quant_fp8(x: np.ndarray, group_size: int, eps: float = 1e-10):
    """x float [..., K] -> (codes uint8 [..., K], scales float32 [..., K/g])."""
    shp = x.shape
    K = shp[-1]
    xf = x.astype(np.float32).reshape(-1, K // group_size, group_size)
    absmax = np.maximum(np.max(np.abs(xf), axis=-1), np.float32(eps)).astype(np.float32)
    s = (absmax / np.float32(FP8_MAX)).astype(np.float32)
    y = (xf / s[..., None]).astype(np.float32)
    y = np.clip(y, -FP8_MAX, FP8_MAX)
    q = to_e4m3fn(y).reshape(shp)
    return q, s.reshape(shp[:-1] + (K // group_size,))


def per_token_quant_fp8(x: np.ndarray, eps: float = 1e-10):
    """Dynamic per-token fp8 (csrc/src/dynamic_per_token_scaled_fp8_quant.cpp;
    ``scale_ub`` is ignored there, :32-34): scale float32 [..., 1]."""
    q, s = per_token_group_quant_fp8(x, x.shape[-1], eps)
    return q, s


def block_fp8_gemm(a_codes, a_scale, b_codes, b_scale, block=(128, 128), bias=None):
    """a_codes uint8 [M, K], a_scale f32 [M, K/bk]; b_codes uint8 [N, K],
    b_scale f32 [ceil(N/bn), K/bk] -> float32 [M, N].

    Per K-block the fp8 products are accumulated in float32, scaled by
    ``a_scale[m, kb] * b_scale[n // bn, kb]`` and added to the running float32
    sum (native_vllm.h:236-255 gives the shapes)."""
    bn, bk = block
    M, K = a_codes.shape
    N = b_codes.shape[0]
    a = torch.from_numpy(from_e4m3fn(a_codes))
    b = torch.from_numpy(from_e4m3fn(b_codes))
    out = torch.zeros(M, N, dtype=torch.float32)
    bs_full = torch.from_numpy(np.repeat(b_scale.astype(np.float32), bn, axis=0)[:N])
    as_t = torch.from_numpy(a_scale.astype(np.float32))
    for kb in range(K // bk):
        part = a[:, kb * bk:(kb + 1) * bk] @ b[:, kb * bk:(kb + 1) * bk].T
        out += part * as_t[:, kb:kb + 1] * bs_full[:, kb][None, :]
    res = out.numpy()
    if bias is not None:
        res = res + bias.astype(np.float32)[None, :]
    return res


def scaled_fp8_mm(a_codes, a_scale, b_codes, b_scale, bias=None):
    """fp8 x fp8 with the scales outside the K sum: a_codes uint8 [M, K], b_codes uint8 [N, K] (the
    operator's weight argument is its [K, N] view); a_scale scalar, [1], [M] or [M, 1]; b_scale scalar,
    [1], [N] or [N, 1] (cutlass_scaled_mm.cpp:23-32 unsqueezes a 0-d x_scale and squeezes an [N, 1]
    w_scale) -> float32 [M, N] = ``(float32 sum over K) * a_scale * b_scale (+ bias)``, formed as
    ``(acc * a_scale) * b_scale`` like the int8 epilogue."""
    a = torch.from_numpy(from_e4m3fn(a_codes))
    b = torch.from_numpy(from_e4m3fn(b_codes))
    acc = (a @ b.T).numpy()
    xs = np.asarray(a_scale, dtype=np.float32).reshape(-1, 1)
    ws = np.asarray(b_scale, dtype=np.float32).reshape(1, -1)
    out = (acc * xs).astype(np.float32) * ws
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.float32).reshape(1, -1)
    return out.astype(np.float32)
