"""Helpers for the GPU parity tests: move numpy data to the device and call the C ABI
through the thrust_amd harness.

The tests name the device and its stream through this module only (DEVICE, stream_handle,
synchronize, empty_cache), so that a session without a GPU can point them at the emulated build of
the kernels (tests/conftest.py does that when THRUST_CDNA4_EMULATED=1)."""
import ctypes

import numpy as np
import torch

DEVICE = "cuda"


def dev(a):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a).cuda() if a.size else torch.empty(0, dtype=torch.from_numpy(a).dtype,
                                                                device="cuda")


def host(t):
    return t.cpu().numpy()


def stream_handle():
    """The current stream as the void* the C ABI takes."""
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def synchronize():
    torch.cuda.synchronize()


def empty_cache():
    torch.cuda.empty_cache()


def memory_allocated():
    return torch.cuda.memory_allocated()
