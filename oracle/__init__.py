"""ctypes binding of the CPU oracle (oracle/oracle.c).

Test infrastructure only: imported by tests/, by the smoke check and by the cpu_baseline
leg of bench.py.  The product package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

DTYPES = {
    np.dtype(np.int8): 0, np.dtype(np.uint8): 1, np.dtype(np.int16): 2,
    np.dtype(np.uint16): 3, np.dtype(np.int32): 4, np.dtype(np.uint32): 5,
    np.dtype(np.int64): 6, np.dtype(np.uint64): 7, np.dtype(np.float32): 8,
    np.dtype(np.float64): 9,
}
OPS = {"plus": 0, "multiplies": 1, "maximum": 2, "minimum": 3}


def build(force=False):
    """Compile liboracle.so with gcc (seconds)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.oracle_sort_keys.argtypes = [i32, vp, i64, i32]
        L.oracle_sort_pairs.argtypes = [i32, vp, i32, vp, i64, i32]
        L.oracle_scan.argtypes = [i32, i32, i32, vp, vp, i64, vp]
        L.oracle_scan_by_key.argtypes = [i32, i32, i32, i32, vp, vp, vp, i64, vp]
        L.oracle_reduce_by_key.argtypes = [i32, i32, i32, vp, vp, vp, vp, i64]
        L.oracle_reduce_by_key.restype = i64
        L.oracle_histogram_even.argtypes = [i32, vp, i64, vp, i32, ctypes.c_double,
                                            ctypes.c_double]
        L.oracle_omp_sort.argtypes = [i32, vp, vp, i64, i32]
        L.oracle_omp_max_threads.restype = i32
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with code {rc}")


def sort_keys(keys, descending=False):
    out = np.ascontiguousarray(keys).copy()
    _check(lib().oracle_sort_keys(DTYPES[out.dtype], _p(out), out.size, int(descending)),
           "sort_keys")
    return out


def sort_pairs(keys, values, descending=False):
    k = np.ascontiguousarray(keys).copy()
    v = np.ascontiguousarray(values).copy()
    assert k.size == v.size
    _check(lib().oracle_sort_pairs(DTYPES[k.dtype], _p(k), v.dtype.itemsize, _p(v), k.size,
                                   int(descending)), "sort_pairs")
    return k, v


def _init_arg(init, dtype):
    if init is None:
        return None, None
    box = np.array([init], dtype=dtype)
    return box, _p(box)


def scan(x, op="plus", exclusive=False, init=None, inplace=False):
    x = np.ascontiguousarray(x)
    out = x.copy() if inplace else np.empty_like(x)
    src = out if inplace else x
    box, ip = _init_arg(init, x.dtype)
    _check(lib().oracle_scan(DTYPES[x.dtype], OPS[op], int(exclusive), _p(src), _p(out),
                             x.size, ip), "scan")
    return out


def scan_by_key(keys, values, op="plus", exclusive=False, init=None):
    keys = np.ascontiguousarray(keys)
    values = np.ascontiguousarray(values)
    out = np.empty_like(values)
    box, ip = _init_arg(init, values.dtype)
    _check(lib().oracle_scan_by_key(DTYPES[keys.dtype], DTYPES[values.dtype], OPS[op],
                                    int(exclusive), _p(keys), _p(values), _p(out),
                                    keys.size, ip), "scan_by_key")
    return out


def reduce_by_key(keys, values, op="plus"):
    keys = np.ascontiguousarray(keys)
    values = np.ascontiguousarray(values)
    ko = np.empty_like(keys)
    vo = np.empty_like(values)
    r = lib().oracle_reduce_by_key(DTYPES[keys.dtype], DTYPES[values.dtype], OPS[op],
                                   _p(keys), _p(values), _p(ko), _p(vo), keys.size)
    if r < 0:
        raise RuntimeError(f"oracle reduce_by_key failed with code {r}")
    return ko[:r].copy(), vo[:r].copy()


def histogram_even(samples, num_bins, lower, upper):
    samples = np.ascontiguousarray(samples)
    counts = np.empty(num_bins, dtype=np.uint32)
    _check(lib().oracle_histogram_even(DTYPES[samples.dtype], _p(samples), samples.size,
                                       _p(counts), num_bins, float(lower), float(upper)),
           "histogram_even")
    return counts


def omp_max_threads():
    return lib().oracle_omp_max_threads()


def omp_sort(keys, values=None, threads=0):
    """In place; restates the reference's OpenMP sort (tile sort + pairwise merges)."""
    assert keys.flags.c_contiguous
    vp = None
    if values is not None:
        assert values.dtype == np.uint32 and values.flags.c_contiguous
        vp = _p(values)
    _check(lib().oracle_omp_sort(DTYPES[keys.dtype], _p(keys), vp, keys.size, threads),
           "omp_sort")
