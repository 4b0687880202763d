"""Small helpers for the GPU tests: device buffers through torch (plumbing only), raw pointers
and the current stream handed to the C ABI."""
import ctypes

import numpy as np
import torch

_SIGNED = {np.dtype(np.uint8): np.uint8, np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32,
           np.dtype(np.uint64): np.int64}


def to_dev(a):
    """numpy array -> device tensor with the same bytes (unsigned types travel as signed)."""
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a.view(_SIGNED.get(a.dtype, a.dtype))).cuda()


def to_host(t, dtype):
    """device tensor -> numpy array reinterpreted as dtype."""
    return t.cpu().numpy().view(dtype)


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def sync():
    torch.cuda.synchronize()


def fetch_async_errors(lib):
    bits = ctypes.c_uint32(0)
    assert lib.ofi_amd_async_error_fetch(ctypes.byref(bits)) == 0
    return bits.value
