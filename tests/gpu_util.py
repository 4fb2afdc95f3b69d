"""Helpers for the GPU parity tests: move numpy data to the device and call the C ABI
through the thrust_amd harness."""
import numpy as np
import torch


def dev(a):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a).cuda() if a.size else torch.empty(0, dtype=torch.from_numpy(a).dtype,
                                                                device="cuda")


def host(t):
    return t.cpu().numpy()
