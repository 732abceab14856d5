"""int4 weight formats and the W4A16 GEMM definition (CPU, numpy).

Test infrastructure only -- never imported by the product package.

Formats restated here:

* GPTQ checkpoint format, ``qweight int32 [K/8, N]`` packed along K and
  ``qzeros int32 [K/g, N/8]`` packed along N with the "+1" convention
  (vllm_gcu/kernels/quantization/rearrange.py:13-29).
* AWQ checkpoint format, ``qweight int32 [K, N/8]`` packed along N with the
  interleave ``[0, 4, 1, 5, 2, 6, 3, 7]`` (rearrange.py:61-101).
* The reference's device layout: ``uint8 [K/2, N]`` "half-group" packing
  (rearrange.py:36-56, 110-128).
* This build's MI355X slab layout (``native_pack``), documented at the
  function.
"""
import numpy as np

AWQ_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)          # rearrange.py:66
# nibble position (within a 32-bit word of the slab layout) of the j-th of the
# 8 consecutive k values a lane feeds to one MFMA step
NATIVE_NIBBLE_OF_J = (0, 4, 1, 5, 2, 6, 3, 7)
SLAB_N = 128
SLAB_K = 128


# ----------------------------------------------------------------------------
# GPTQ checkpoint format
# ----------------------------------------------------------------------------
def gptq_unpack_weight(qweight: np.ndarray) -> np.ndarray:
    """int32 [K/8, N] -> uint8 [K, N]; nibble i of row r is k = 8r + i.

    Follows rearrange.py:13-21 (shift by ``range(0, 32, 4)``, mask 15,
    reshape ``(-1, N)``).
    """
    qw = np.ascontiguousarray(qweight).view(np.uint32)
    shifts = (4 * np.arange(8, dtype=np.uint32)).reshape(1, 8, 1)
    w = (qw[:, None, :] >> shifts) & np.uint32(15)
    return w.reshape(-1, qw.shape[1]).astype(np.uint8)


def gptq_pack_weight(w: np.ndarray) -> np.ndarray:
    """Inverse of :func:`gptq_unpack_weight` (what a GPTQ exporter writes)."""
    K, N = w.shape
    assert K % 8 == 0
    w32 = w.astype(np.uint32).reshape(K // 8, 8, N)
    out = np.zeros((K // 8, N), dtype=np.uint32)
    for i in range(8):
        out |= (w32[:, i, :] & 15) << np.uint32(4 * i)
    return out.view(np.int32)


def gptq_unpack_zeros(qzeros: np.ndarray) -> np.ndarray:
    """int32 [G, N/8] -> uint8 [G, N] with ``z = (stored + 1) & 15``.

    Follows rearrange.py:24-29: nibble j of column c is n = 8c + j, then the
    GPTQ "+1" and a 4-bit mask (so a stored 15 wraps to 0).
    """
    qz = np.ascontiguousarray(qzeros).view(np.uint32)
    shifts = (4 * np.arange(8, dtype=np.uint32)).reshape(1, 1, 8)
    z = (qz[:, :, None] >> shifts) & np.uint32(15)
    z = (z + 1) & np.uint32(15)
    return z.reshape(qz.shape[0], -1).astype(np.uint8)


def gptq_pack_zeros(z: np.ndarray) -> np.ndarray:
    """Logical zero-points uint8 [G, N] -> GPTQ qzeros (stores ``z - 1 mod 16``)."""
    G, N = z.shape
    assert N % 8 == 0
    s = ((z.astype(np.int32) - 1) & 15).astype(np.uint32).reshape(G, N // 8, 8)
    out = np.zeros((G, N // 8), dtype=np.uint32)
    for j in range(8):
        out |= s[:, :, j] << np.uint32(4 * j)
    return out.view(np.int32)


# ----------------------------------------------------------------------------
# AWQ checkpoint format
# ----------------------------------------------------------------------------
def awq_unpack(qx: np.ndarray) -> np.ndarray:
    """int32 [R, N/8] -> uint8 [R, N] for AWQ weights *and* zeros.

    rearrange.py:66-101: nibble i of column c goes to temporary column 8c+i;
    logical column 8c+j then reads temporary column ``8c + AWQ_ORDER[j]``; no
    "+1" on zeros.
    """
    q = np.ascontiguousarray(qx).view(np.uint32)
    shifts = (4 * np.arange(8, dtype=np.uint32)).reshape(1, 1, 8)
    t = (q[:, :, None] >> shifts) & np.uint32(15)        # [R, N/8, 8] temp order
    t = t[:, :, list(AWQ_ORDER)]
    return t.reshape(q.shape[0], -1).astype(np.uint8)


def awq_pack(x: np.ndarray) -> np.ndarray:
    """Inverse of :func:`awq_unpack` (what AutoAWQ writes)."""
    R, N = x.shape
    assert N % 8 == 0
    v = x.astype(np.uint32).reshape(R, N // 8, 8)
    out = np.zeros((R, N // 8), dtype=np.uint32)
    for j in range(8):
        out |= (v[:, :, j] & 15) << np.uint32(4 * AWQ_ORDER[j])
    return out.view(np.int32)


# ----------------------------------------------------------------------------
# Reference device layout (uint8 half-group)
# ----------------------------------------------------------------------------
def ref_halfgroup_pack(w: np.ndarray, rearrange_group: int = 128) -> np.ndarray:
    """uint8 [K, N] (values 0..15) -> uint8 [K/2, N].

    rearrange.py:36-56: with h = rearrange_group/2, row ``G*h + i`` of the
    result holds ``w[G*2h + i]`` in the low nibble and ``w[G*2h + h + i]`` in
    the high nibble, i in [0, h).  K not a multiple of the group is padded
    with zero rows by the reference (rearrange.py:37-43 pads ``K % group``
    rows, which only reaches a multiple when that remainder is group/2; the
    restatement requires K % group == 0, which every caller satisfies).
    """
    K, N = w.shape
    h = rearrange_group // 2
    assert K % rearrange_group == 0
    v = w.reshape(K // rearrange_group, 2, h, N)
    out = (v[:, 0] & 15) | ((v[:, 1] & 15) << 4)
    return out.reshape(K // 2, N).astype(np.uint8)


def ref_halfgroup_unpack(rw: np.ndarray, rearrange_group: int = 128) -> np.ndarray:
    """Inverse of :func:`ref_halfgroup_pack`: uint8 [K/2, N] -> uint8 [K, N]."""
    K2, N = rw.shape
    h = rearrange_group // 2
    v = rw.astype(np.uint8).reshape(K2 // h, h, N)
    out = np.stack([v & 15, v >> 4], axis=1)               # [G, 2, h, N]
    return out.reshape(2 * K2, N)


def rearrange_gptq(qweight, qzeros, scales, rearrange_group=128):
    """Restatement of ``rearrange_uint4_int32_uint8_gptq`` (rearrange.py:6-58).

    Returns ``(rweight uint8 [K/2, N], zeros_f [K/g, N])`` where ``zeros_f =
    z * scales`` evaluated in the dtype of ``scales`` (rearrange.py:33: int8
    zeros are promoted to the scales dtype and multiplied there).
    """
    w = gptq_unpack_weight(qweight)
    rweight = ref_halfgroup_pack(w, rearrange_group)
    zeros_f = None
    if qzeros is not None:
        z = gptq_unpack_zeros(qzeros)
        zeros_f = (z.astype(scales.dtype) * scales).astype(scales.dtype)
    return rweight, zeros_f


def rearrange_awq(qweight, qzeros, scales, rearrange_group=128,
                  zeros_in_int8=False, use_w4a8=False):
    """Restatement of ``rearrange_uint4_int32_uint8_awq`` (rearrange.py:61-133)."""
    w = awq_unpack(qweight).astype(np.int8)
    z = None
    if qzeros is not None:
        z = awq_unpack(qzeros).astype(np.int8)
        if not zeros_in_int8:
            z = (z.astype(scales.dtype) * scales).astype(scales.dtype)
    if use_w4a8:
        w = w - 8
        z = None
    rweight = ref_halfgroup_pack(w.astype(np.uint8) & 15, rearrange_group)
    if zeros_in_int8:
        return rweight.view(np.int8), z
    return rweight, z


# ----------------------------------------------------------------------------
# This build's MI355X slab layout
# ----------------------------------------------------------------------------
def native_pack(w: np.ndarray) -> np.ndarray:
    """uint8 [K, N] (0..15) -> int32 [K/8, N] holding the slab layout.

    The flat int32 stream is ``[N/128 slabs][K/128 groups][8 tiles][64 lanes]
    [4 words]``.  Word ``s`` of lane ``l`` (c = l % 16, kq = l // 16) of tile
    ``t`` in (slab S, group g) holds, in nibble ``NATIVE_NIBBLE_OF_J[j]``, the
    weight at ``k = 128 g + 32 s + 8 kq + j`` and ``n = 128 S + 8 c + t``.
    A wavefront therefore reads one tile as a single contiguous 1 KiB
    (64 lanes x 16 B), each lane's word ``s`` is its B operand for MFMA step
    ``s`` of the group, and the 8 columns a lane owns across the 8 tiles are
    contiguous in the output row.
    """
    K, N = w.shape
    assert K % SLAB_K == 0 and N % SLAB_N == 0
    # v[g, s, kq, j, S, c, t]
    v = w.astype(np.uint32).reshape(K // 128, 4, 4, 8, N // 128, 16, 8)
    words = np.zeros((N // 128, K // 128, 8, 4, 16, 4), dtype=np.uint32)  # S,g,t,kq,c,s
    for j in range(8):
        # v[:, :, :, j] -> [g, s, kq, S, c, t] -> [S, g, t, kq, c, s]
        part = v[:, :, :, j].transpose(3, 0, 5, 2, 4, 1)
        words |= (part & 15) << np.uint32(4 * NATIVE_NIBBLE_OF_J[j])
    return words.reshape(K // 8, N).view(np.int32)


def native_unpack(packed: np.ndarray, K: int, N: int) -> np.ndarray:
    """Inverse of :func:`native_pack`, written as a scalar index walk."""
    flat = np.ascontiguousarray(packed).view(np.uint32).reshape(-1)
    w = np.zeros((K, N), dtype=np.uint8)
    idx = 0
    for S in range(N // 128):
        for g in range(K // 128):
            for t in range(8):
                for lane in range(64):
                    c, kq = lane % 16, lane // 16
                    for s in range(4):
                        word = int(flat[idx]); idx += 1
                        for j in range(8):
                            nib = (word >> (4 * NATIVE_NIBBLE_OF_J[j])) & 15
                            w[128 * g + 32 * s + 8 * kq + j, 128 * S + 8 * c + t] = nib
    return w


def native_pack_zeros(z: np.ndarray) -> np.ndarray:
    """Logical zero-points uint8 [G, N] -> int32 [G, N/8]; nibble j of column
    c is ``z[g, 8c + j]`` (true value, no "+1" convention)."""
    G, N = z.shape
    v = z.astype(np.uint32).reshape(G, N // 8, 8)
    out = np.zeros((G, N // 8), dtype=np.uint32)
    for j in range(8):
        out |= (v[:, :, j] & 15) << np.uint32(4 * j)
    return out.view(np.int32)


# ----------------------------------------------------------------------------
# W4A16 GEMM definition
# ----------------------------------------------------------------------------
def dequantize(q: np.ndarray, z: np.ndarray, s: np.ndarray, group_size: int) -> np.ndarray:
    """``w[k, n] = (q[k, n] - z[k // g, n]) * s[k // g, n]`` in float32.

    q uint8 [K, N]; z integer [K/g, N] (or None -> 8, the symmetric int4
    default); s float [K/g, N].  This is the dequantization the operators
    gptq_gemm_gcu / awq_gemm_gcu are defined by (csrc/src/gptq_gemm_gcu.cpp:27-48
    hands ``(out, x, qweight, scale, zeros, bias, group_size)`` to the vendor
    GEMM).
    """
    K, N = q.shape
    g = K if group_size in (-1, 0) else group_size
    zi = np.full((K // g, N), 8, np.float32) if z is None else z.astype(np.float32)
    w = q.astype(np.float32).reshape(K // g, g, N)
    w -= zi[:, None, :]                    # in place: the same two roundings, no full-size temporaries
    w *= s.astype(np.float32)[:, None, :]
    return w.reshape(K, N)


def dequantize_prescaled_zeros(q, zs, s, group_size):
    """``w = q * s - zs`` with ``zs = z * s`` pre-multiplied in the scale dtype,
    the form the reference's GPTQ loader hands to the device
    (rearrange.py:33-34)."""
    K, N = q.shape
    g = K if group_size in (-1, 0) else group_size
    qf = q.astype(np.float32).reshape(K // g, g, N)
    w = qf * s.astype(np.float32)[:, None, :] - zs.astype(np.float32)[:, None, :]
    return w.reshape(K, N)


def w4a16_gemm(x: np.ndarray, q, z, s, group_size: int, bias=None) -> np.ndarray:
    """Oracle for the W4A16 GEMM: float32 result of
    ``x.float() @ dequantize(q, z, s)`` (+ bias); the caller casts to the
    activation dtype.  x is float16 or a float32 array holding bfloat16
    values."""
    import torch
    w = dequantize(q, z, s, group_size)
    out = torch.matmul(torch.from_numpy(np.ascontiguousarray(x.astype(np.float32))),
                       torch.from_numpy(np.ascontiguousarray(w))).numpy()
    if bias is not None:
        out = out + bias.astype(np.float32)[None, :]
    return out
