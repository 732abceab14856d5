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


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Zero-initialised scratch for split-K partial tiles and arrival counters.
    One buffer per (device, stream) so launches that may overlap never share
    it; the kernels restore the counters to zero themselves."""
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        size = max(nbytes, 8 << 20)
        buf = torch.zeros(size, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf
