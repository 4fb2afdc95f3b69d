"""Python mirror of the Thrust calls on the hot path, over torch device tensors.

Argument meaning follows the reference's public API (thrust/sort.h, thrust/scan.h,
thrust/reduce.h); every function goes through the two-phase C ABI: size query, temporary
storage from torch's caching allocator, run on torch's current stream.
"""
import ctypes

import numpy as np
import torch

from . import capi

_DT = {
    torch.int8: capi.I8, torch.uint8: capi.U8, torch.int16: capi.I16, torch.int32: capi.I32,
    torch.int64: capi.I64, torch.float32: capi.F32, torch.float64: capi.F64,
}
for _name, _code in (("uint16", capi.U16), ("uint32", capi.U32), ("uint64", capi.U64)):
    if hasattr(torch, _name):
        _DT[getattr(torch, _name)] = _code

_NP = {
    capi.I8: np.int8, capi.U8: np.uint8, capi.I16: np.int16, capi.U16: np.uint16,
    capi.I32: np.int32, capi.U32: np.uint32, capi.I64: np.int64, capi.U64: np.uint64,
    capi.F32: np.float32, capi.F64: np.float64,
}
_OPS = {"plus": capi.PLUS, "multiplies": capi.MULTIPLIES, "maximum": capi.MAXIMUM,
        "minimum": capi.MINIMUM}


def dtype_code(t):
    return _DT[t.dtype]


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() else ctypes.c_void_p(
        t.data_ptr() if t is not None else 0)


def _need_cuda(*ts):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("device tensors required: there is no CPU path")
        if not t.is_contiguous():
            raise ValueError("contiguous tensors required")


def _temp(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def _init_box(init, code):
    if init is None:
        return None, ctypes.c_void_p(0)
    box = np.array([init], dtype=_NP[code])
    return box, box.ctypes.data_as(ctypes.c_void_p)


def sort(keys, descending=False):
    """thrust::sort(keys.begin(), keys.end()[, thrust::greater<T>()]) — in place."""
    _need_cuda(keys)
    L = capi.lib()
    nb = ctypes.c_size_t(0)
    code = dtype_code(keys)
    n = keys.numel()
    capi.check(L.thrust_cdna4_sort_keys(None, ctypes.byref(nb), code, _ptr(keys), n,
                                        int(descending), _stream()), "sort_keys(size)")
    tmp = _temp(nb.value, keys.device)
    capi.check(L.thrust_cdna4_sort_keys(_ptr(tmp), ctypes.byref(nb), code, _ptr(keys), n,
                                        int(descending), _stream()), "sort_keys")
    # thrust::sort(thrust::device, ...) returns when the work is done and throws if it failed
    capi.check(L.thrust_cdna4_sort_status(_ptr(tmp), n, _stream()), "sort_keys: a wait inside the sort did not end")
    return keys


def sort_by_key(keys, values, descending=False):
    """thrust::sort_by_key(keys.begin(), keys.end(), values.begin()[, greater]) — in place."""
    _need_cuda(keys, values)
    if keys.numel() != values.numel():
        raise ValueError("keys and values differ in length")
    L = capi.lib()
    nb = ctypes.c_size_t(0)
    code = dtype_code(keys)
    n = keys.numel()
    vb = values.element_size()
    capi.check(L.thrust_cdna4_sort_pairs(None, ctypes.byref(nb), code, _ptr(keys), vb,
                                         _ptr(values), n, int(descending), _stream()),
               "sort_pairs(size)")
    tmp = _temp(nb.value, keys.device)
    capi.check(L.thrust_cdna4_sort_pairs(_ptr(tmp), ctypes.byref(nb), code, _ptr(keys), vb,
                                         _ptr(values), n, int(descending), _stream()),
               "sort_pairs")
    capi.check(L.thrust_cdna4_sort_status(_ptr(tmp), n, _stream()), "sort_pairs: a wait inside the sort did not end")
    return keys, values


def _scan(x, out, op, exclusive, init):
    _need_cuda(x, out)
    if out is None:
        out = torch.empty_like(x)
    if out.dtype != x.dtype or out.numel() != x.numel():
        raise ValueError("output must match input in dtype and length")
    L = capi.lib()
    code = dtype_code(x)
    nb = ctypes.c_size_t(0)
    box, ip = _init_box(init, code)
    n = x.numel()
    capi.check(L.thrust_cdna4_scan(None, ctypes.byref(nb), code, _OPS[op], int(exclusive),
                                   _ptr(x), _ptr(out), n, ip, _stream()), "scan(size)")
    tmp = _temp(nb.value, x.device)
    capi.check(L.thrust_cdna4_scan(_ptr(tmp), ctypes.byref(nb), code, _OPS[op], int(exclusive),
                                   _ptr(x), _ptr(out), n, ip, _stream()), "scan")
    return out


def inclusive_scan(x, out=None, op="plus"):
    """thrust::inclusive_scan(x.begin(), x.end(), out.begin(), op); out may be x."""
    return _scan(x, out, op, False, None)


def exclusive_scan(x, out=None, init=None, op="plus"):
    """thrust::exclusive_scan(x.begin(), x.end(), out.begin(), init, op); out may be x."""
    return _scan(x, out, op, True, init)


def _scan_by_key(keys, values, out, op, exclusive, init):
    _need_cuda(keys, values, out)
    if out is None:
        out = torch.empty_like(values)
    if keys.numel() != values.numel() or out.numel() != values.numel() or out.dtype != values.dtype:
        raise ValueError("keys, values and output must match in length (and value dtype)")
    L = capi.lib()
    kc, vc = dtype_code(keys), dtype_code(values)
    nb = ctypes.c_size_t(0)
    box, ip = _init_box(init, vc)
    n = keys.numel()
    args = (kc, vc, _OPS[op], int(exclusive), _ptr(keys), _ptr(values), _ptr(out), n, ip, _stream())
    capi.check(L.thrust_cdna4_scan_by_key(None, ctypes.byref(nb), *args), "scan_by_key(size)")
    tmp = _temp(nb.value, keys.device)
    capi.check(L.thrust_cdna4_scan_by_key(_ptr(tmp), ctypes.byref(nb), *args), "scan_by_key")
    return out


def inclusive_scan_by_key(keys, values, out=None, op="plus"):
    return _scan_by_key(keys, values, out, op, False, None)


def exclusive_scan_by_key(keys, values, out=None, init=None, op="plus"):
    return _scan_by_key(keys, values, out, op, True, init)


def reduce_by_key(keys, values, keys_out=None, values_out=None, op="plus"):
    """thrust::reduce_by_key; returns (keys_out[:r], values_out[:r]) like the iterator pair."""
    _need_cuda(keys, values, keys_out, values_out)
    if keys.numel() != values.numel():
        raise ValueError("keys and values differ in length")
    if keys_out is None:
        keys_out = torch.empty_like(keys)
    if values_out is None:
        values_out = torch.empty_like(values)
    L = capi.lib()
    kc, vc = dtype_code(keys), dtype_code(values)
    nb = ctypes.c_size_t(0)
    n = keys.numel()
    nruns = torch.zeros(1, dtype=torch.int64, device=keys.device)
    args = (kc, vc, _OPS[op], _ptr(keys), _ptr(values), _ptr(keys_out), _ptr(values_out),
            _ptr(nruns), n, _stream())
    capi.check(L.thrust_cdna4_reduce_by_key(None, ctypes.byref(nb), *args), "reduce_by_key(size)")
    tmp = _temp(nb.value, keys.device)
    capi.check(L.thrust_cdna4_reduce_by_key(_ptr(tmp), ctypes.byref(nb), *args), "reduce_by_key")
    r = int(nruns.item())  # synchronises, as the reference does (reduce_by_key.h:1049-1052)
    return keys_out[:r], values_out[:r]


def histogram_even(samples, num_bins, lower, upper, counts=None):
    _need_cuda(samples, counts)
    if counts is None:
        counts = torch.empty(num_bins, dtype=torch.int32, device=samples.device)
    if counts.numel() != num_bins or counts.element_size() != 4:
        raise ValueError("counts must hold num_bins 32-bit counters")
    L = capi.lib()
    nb = ctypes.c_size_t(0)
    args = (dtype_code(samples), _ptr(samples), samples.numel(), _ptr(counts), int(num_bins),
            float(lower), float(upper), _stream())
    capi.check(L.thrust_cdna4_histogram_even(None, ctypes.byref(nb), *args), "histogram(size)")
    tmp = _temp(nb.value, samples.device)
    capi.check(L.thrust_cdna4_histogram_even(_ptr(tmp), ctypes.byref(nb), *args), "histogram")
    return counts
