"""int4 weight repack at load time, on the device.

Counterpart of vllm_gcu/kernels/quantization/rearrange.py:6-133.  The
reference unpacks GPTQ / AWQ checkpoints on the CPU into a ``uint8 [K/2, N]``
half-group layout for the GCU; here the same checkpoints (or tensors already in
the reference layout) are converted by HIP kernels into the MI355X slab layout
the W4A16 kernels stream (see include/mi355q.h), and zero-points are kept as
packed int4 instead of being pre-multiplied by the scales.
"""
import weakref

import torch

from .. import _runtime as rt
from ... import _lib


def _repack(src: torch.Tensor, fmt: int, batch: int, K: int, N: int) -> torch.Tensor:
    rt.require_gpu(src)
    src = src.contiguous()
    shape = (K // 8, N) if batch is None else (batch, K // 8, N)
    dst = torch.empty(shape, dtype=torch.int32, device=src.device)
    with torch.cuda.device(src.device):
        _lib.call("mi355q_w4_repack", src.data_ptr(), fmt, dst.data_ptr(),
                  1 if batch is None else batch, K, N, rt.stream_ptr())
    return dst


def _repack_zeros(src: torch.Tensor, fmt: int) -> torch.Tensor:
    rt.require_gpu(src)
    src = src.contiguous()
    assert src.dtype == torch.int32
    batch = 1 if src.dim() == 2 else src.shape[0]
    G, N8 = src.shape[-2], src.shape[-1]
    dst = torch.empty_like(src)
    with torch.cuda.device(src.device):
        _lib.call("mi355q_w4_repack_zeros", src.data_ptr(), fmt, dst.data_ptr(), batch, G, N8 * 8,
                  rt.stream_ptr())
    return dst


def rearrange_uint4_int32_gptq(qweight: torch.Tensor, qzeros, scales=None):
    """GPTQ checkpoint tensors -> (slab-layout qweight int32 [K/8, N], packed
    zero-points int32 [K/g, N/8] with the "+1" applied).

    qweight int32 [K/8, N] (or [E, K/8, N]); qzeros int32 [K/g, N/8] or None.
    Same inputs as rearrange_uint4_int32_uint8_gptq (rearrange.py:6-58).
    """
    assert qweight.dtype == torch.int32
    batch = None if qweight.dim() == 2 else qweight.shape[0]
    K, N = qweight.shape[-2] * 8, qweight.shape[-1]
    w = _repack(qweight, _lib.W4_SRC_GPTQ, batch, K, N)
    z = None if qzeros is None else _repack_zeros(qzeros, _lib.W4_SRC_GPTQ)
    return w, z


def rearrange_uint4_int32_awq(qweight: torch.Tensor, qzeros, scales=None):
    """AWQ checkpoint tensors (qweight int32 [K, N/8], qzeros int32 [K/g, N/8])
    -> (slab-layout qweight, packed zero-points).  Same inputs as
    rearrange_uint4_int32_uint8_awq (rearrange.py:61-133)."""
    assert qweight.dtype == torch.int32
    batch = None if qweight.dim() == 2 else qweight.shape[0]
    K, N = qweight.shape[-2], qweight.shape[-1] * 8
    w = _repack(qweight, _lib.W4_SRC_AWQ, batch, K, N)
    z = None if qzeros is None else _repack_zeros(qzeros, _lib.W4_SRC_AWQ)
    return w, z


def from_reference_layout(rweight: torch.Tensor, transposed: bool = False) -> torch.Tensor:
    """Reference device layout -> slab layout.

    ``rweight`` is uint8/int8 ``[K/2, N]`` (dense, rearrange.py:44-56) or, with
    ``transposed=True``, ``[N, K/2]`` / ``[E, N, K/2]`` (MoE experts,
    moe_wna16.py:464-466).  The result keeps the GPTQ checkpoint shape
    ``[K/8, N]`` (``[E, K/8, N]``), dtype int32.
    """
    assert rweight.dtype in (torch.uint8, torch.int8)
    batch = None if rweight.dim() == 2 else rweight.shape[0]
    if transposed:
        N, K = rweight.shape[-2], rweight.shape[-1] * 2
        fmt = _lib.W4_SRC_REF_NK
    else:
        K, N = rweight.shape[-2] * 2, rweight.shape[-1]
        fmt = _lib.W4_SRC_REF_KN
    return _repack(rweight, fmt, batch, K, N)


def from_reference_w4a8(rweight: torch.Tensor) -> torch.Tensor:
    """The reference's w4a8 expert tensor -> slab layout int32 [E, K/8, N].

    ``rweight`` is int8 with shape [E, N, K/2] whose memory is [E, K/2, N]
    (w4a8.py:199-220 permutes, makes contiguous and then only *views* the
    transposed shape; fused_moe_quant_kernel_ex.cpp:37 views it back), bytes in
    half-groups of 32 rows holding ``w - 8`` as signed nibbles (rearrange.py:
    61-133 with ``use_w4a8``, ``rearrange_group=64``).  The slab tensor holds the
    unsigned ``w`` with the implicit zero-point 8."""
    assert rweight.dtype in (torch.int8, torch.uint8) and rweight.dim() == 3
    E, N, K2 = rweight.shape
    return _repack(rweight, _lib.W4_SRC_REF_KN_G64S, E, 2 * K2, N)


def pack_int8_zeros(z: torch.Tensor) -> torch.Tensor:
    """int8/uint8 zero-points [..., G, N] (the AWQ ``zeros_in_int8`` form,
    awq.py:80-106) -> packed int32 [..., G, N/8]."""
    v = z.to(torch.int32) & 15
    v = v.reshape(*z.shape[:-1], z.shape[-1] // 8, 8)
    shifts = torch.arange(0, 32, 4, device=z.device, dtype=torch.int32)
    return (v << shifts).sum(dim=-1).to(torch.int32)


def unpack_slab(packed: torch.Tensor) -> torch.Tensor:
    """Slab layout int32 [K/8, N] -> uint8 [K, N], one int4 value per byte
    (parity/debug helper)."""
    rt.require_gpu(packed)
    assert packed.dtype == torch.int32
    batch = None if packed.dim() == 2 else packed.shape[0]
    K, N = packed.shape[-2] * 8, packed.shape[-1]
    shape = (K, N) if batch is None else (batch, K, N)
    dst = torch.empty(shape, dtype=torch.uint8, device=packed.device)
    with torch.cuda.device(packed.device):
        _lib.call("mi355q_w4_unpack", packed.contiguous().data_ptr(), dst.data_ptr(),
                  1 if batch is None else batch, K, N, rt.stream_ptr())
    return dst


# kslab allocations by (device index, address) -> byte size: the flag has to survive views
# (``weight.t()`` is what the int8 operators receive), which drop Python attributes
_KSLAB_ALLOCS = {}           # (device, address) -> [bytes, live tensor objects that carry the flag]


def _unregister_kslab(key) -> None:
    ent = _KSLAB_ALLOCS.get(key)
    if ent is not None:
        ent[1] -= 1
        if ent[1] <= 0:
            del _KSLAB_ALLOCS[key]


def _register_kslab(t: torch.Tensor) -> None:
    """Entries live as long as a flagged tensor object on that memory does (the tensor made by
    to_kslab, a Parameter wrapped around it and marked with mark_kslab, ...)."""
    key = (t.device.index, t.data_ptr())
    ent = _KSLAB_ALLOCS.setdefault(key, [t.numel() * t.element_size(), 0])
    ent[0] = t.numel() * t.element_size()
    ent[1] += 1
    weakref.finalize(t, _unregister_kslab, key)


def is_kslab(w: torch.Tensor) -> bool:
    """True for a tensor made by :func:`to_kslab`, for a Parameter / view marked with
    :func:`mark_kslab`, and for any view that starts at the address of such an allocation and
    covers all of it (e.g. ``w.t()``)."""
    if getattr(w, "_mi355q_kslab", False):
        return True
    ent = _KSLAB_ALLOCS.get((w.device.index, w.data_ptr())) if w.is_cuda else None
    return ent is not None and ent[0] == w.numel() * w.element_size()


def kslab_eligible(w: torch.Tensor) -> bool:
    return (w.dim() in (2, 3) and w.element_size() in (1, 2) and w.shape[-2] % 64 == 0
            and w.shape[-1] % 128 == 0 and w.is_contiguous())


def to_kslab(w: torch.Tensor) -> torch.Tensor:
    """K-contiguous weights ``[N, K]`` / ``[E, N, K]`` (fp8, int8 or 16-bit) ->
    the same bytes in the streaming "kslab" order (see include/mi355q.h); the
    result keeps shape and dtype and carries the attribute ``_mi355q_kslab``.
    The reference keeps these weights row-major (fp8.py:72-166, w8a8.py:240-262);
    this is a load-time conversion of this build, like its int4 rearrange."""
    rt.require_gpu(w)
    if is_kslab(w):
        return w
    if not kslab_eligible(w):
        raise RuntimeError(f"to_kslab: need contiguous [.., N % 64 == 0, K % 128 == 0] 1- or 2-byte weights, "
                           f"got {w.dtype} {tuple(w.shape)}")
    batch = 1 if w.dim() == 2 else w.shape[0]
    dst = torch.empty_like(w)
    with torch.cuda.device(w.device):
        _lib.call("mi355q_kslab_repack", w.data_ptr(), dst.data_ptr(), batch, w.shape[-2], w.shape[-1],
                  w.element_size(), rt.stream_ptr())
    dst._mi355q_kslab = True
    _register_kslab(dst)
    return dst


def mark_kslab(p: torch.Tensor) -> torch.Tensor:
    """Re-attach the layout flag after wrapping a kslab tensor (e.g. in a Parameter)."""
    p._mi355q_kslab = True
    _register_kslab(p)
    return p


def kslab_parameters_(layer, names) -> None:
    """Load-time, in place: replace each named parameter of ``layer`` that
    qualifies by its kslab-ordered copy (the row-major tensor is dropped, so no
    weight is resident twice)."""
    for name in names:
        w = getattr(layer, name, None)
        if w is None or is_kslab(w) or not w.is_cuda or not kslab_eligible(w.data):
            continue
        packed = torch.nn.Parameter(to_kslab(w.data), requires_grad=False)
        setattr(layer, name, mark_kslab(packed))
