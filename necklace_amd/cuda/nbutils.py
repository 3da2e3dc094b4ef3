"""Device helpers with the names of necklace/cuda/nbutils.py:11-39, on PyTorch-ROCm.

numba is gone: a "device array" is a torch tensor on the GPU, a "stream" is a
torch.cuda.Stream (a HIP stream).
"""
import ctypes as ctp

import numpy as np
import torch


def cuda_select_device(dev_i):
    """necklace/cuda/nbutils.py:11-17."""
    torch.cuda.set_device(int(dev_i))


def cuda_current_context():
    """necklace/cuda/nbutils.py:20-22; HIP has no user-visible context object, the device is it."""
    return torch.device("cuda", torch.cuda.current_device())


def cuda_stream():
    """necklace/cuda/nbutils.py:25-27: a new stream (default priority)."""
    return torch.cuda.Stream()


def cuda_to_device(A, stream=None):
    """necklace/cuda/nbutils.py:30-34: copy a host array to the current GPU."""
    if isinstance(A, torch.Tensor):
        t = A
    else:
        t = torch.from_numpy(np.ascontiguousarray(A))
    if stream is None:
        return t.to("cuda")
    with torch.cuda.stream(stream):
        return t.to("cuda", non_blocking=False)


def cuda_devarr_c_void_p(d_arr):
    """necklace/cuda/nbutils.py:37-39: device address as ctypes.c_void_p."""
    return ctp.c_void_p(d_arr.data_ptr())


# torch's accessor for the raw handle of the current stream (no Stream object is built: 0.3 us
# against 1.9 us); absent in some builds, then the documented route is taken
_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_handle(stream=None, device=None):
    """hipStream_t (as int) of `stream`; None means torch's current stream on `device`."""
    if stream is None:
        if _raw_current_stream is not None:
            index = device if isinstance(device, int) else getattr(device, "index", None)
            if index is not None:
                return _raw_current_stream(index)
        return torch.cuda.current_stream(device).cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream
