"""Small runtime helpers shared by the operator wrappers: stream handle,
dtype codes, the per-(device, stream) split-K workspace."""
import torch

from .. import _lib

_DT = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}") from None


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mi355q operators need tensors on the GPU; got a "
                               f"{t.device} tensor (there is no CPU fallback)")


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def ptr(t):
    return 0 if t is None else t.data_ptr()


_workspaces = {}
_retired = []          # superseded buffers: a captured graph may still hold their addresses
# the largest plan of any entry point: two split-K regions of 64 MiB, arrival counters, slack
WORKSPACE_BYTES = (130 << 20)


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Zero-initialised scratch for split-K partial tiles and arrival counters.
    One buffer per (device, stream) so launches that may overlap never share
    it; the kernels restore the counters to zero themselves.

    The buffer is allocated once at the size of the largest plan, so its
    address never changes afterwards: a HIP graph captured on the stream keeps
    pointing at live memory whatever runs eagerly later.  Should a larger
    request ever arrive, the old buffer is kept alive (never handed back to the
    allocator) for the same reason.  Allocating or growing while the stream is
    being captured raises: the allocation and its zero fill would land in the
    graph's private pool.  Run the operator once on the capture stream first."""
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                "mi355q: the split-K workspace of this stream would have to be allocated during graph "
                f"capture ({nbytes} bytes asked, {0 if buf is None else buf.numel()} held); run the "
                "operator once on the capture stream before capturing")
        if buf is not None:
            _retired.append(buf)
        buf = torch.zeros(max(nbytes, WORKSPACE_BYTES), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf
