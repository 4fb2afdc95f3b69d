"""CPU-only checks of the C-ABI boundary: the library loads without a GPU, exports every
symbol include/thrust_cdna4.h declares, answers temporary-storage size queries (which touch
no device) and rejects bad arguments with an error code instead of crashing."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from thrust_amd import capi


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "thrust_cdna4.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(thrust_cdna4_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(capi.SYMBOLS)


def test_library_exports_every_declared_symbol():
    L = capi.lib()
    for name in declared_symbols():
        assert hasattr(L, name), name
    assert L.thrust_cdna4_abi_version() == 1


def _size(fn, *args):
    nb = ctypes.c_size_t(0)
    rc = fn(None, ctypes.byref(nb), *args)
    return rc, nb.value


def test_size_queries_need_no_device():
    L = capi.lib()
    n = 1 << 20
    rc, b = _size(L.thrust_cdna4_sort_keys, capi.U32, None, n, 0, None)
    assert rc == 0 and b >= 4 * n  # holds the alternate key buffer
    rc, b2 = _size(L.thrust_cdna4_sort_pairs, capi.U64, None, 4, None, n, 0, None)
    assert rc == 0 and b2 >= 12 * n
    rc, b = _size(L.thrust_cdna4_scan, capi.I32, capi.PLUS, 0, None, None, n, None, None)
    assert rc == 0 and 0 < b < n
    rc, b = _size(L.thrust_cdna4_scan_by_key, capi.I32, capi.F32, capi.PLUS, 0, None, None, None, n,
                  None, None)
    assert rc == 0 and 0 < b < n
    rc, b = _size(L.thrust_cdna4_reduce_by_key, capi.I32, capi.I32, capi.PLUS, None, None, None, None,
                  None, n, None)
    assert rc == 0 and 0 < b < n
    rc, b = _size(L.thrust_cdna4_histogram_even, capi.U8, None, n, None, 256, 0.0, 256.0, None)
    assert rc == 0 and b > 0
    # n == 0 is a valid query
    rc, b = _size(L.thrust_cdna4_sort_keys, capi.U32, None, 0, 0, None)
    assert rc == 0


@pytest.mark.parametrize("bad", ["dtype", "negative_n", "op", "value_bytes", "bins", "range", "temp_alignment"])
def test_bad_arguments_return_an_error_code(bad):
    L = capi.lib()
    n = 100
    if bad == "dtype":
        rc, _ = _size(L.thrust_cdna4_sort_keys, 99, None, n, 0, None)
    elif bad == "negative_n":
        rc, _ = _size(L.thrust_cdna4_scan, capi.I32, capi.PLUS, 0, None, None, -1, None, None)
    elif bad == "op":
        rc, _ = _size(L.thrust_cdna4_scan, capi.I32, 17, 0, None, None, n, None, None)
    elif bad == "value_bytes":
        rc, _ = _size(L.thrust_cdna4_sort_pairs, capi.U32, None, 3, None, n, 0, None)
    elif bad == "temp_alignment":
        # the descriptors in the temporary storage are 64-bit atoms: an address that would fault there
        # is refused on the host.  Empty inputs, so that the accepted calls touch no device either.
        import ctypes
        nb = ctypes.c_size_t(1 << 20)

        def calls(temp):
            t = ctypes.c_void_p(temp)
            return [L.thrust_cdna4_sort_keys(t, ctypes.byref(nb), capi.U32, None, 0, 0, None),
                    L.thrust_cdna4_sort_pairs(t, ctypes.byref(nb), capi.U32, None, 4, None, 0, 0, None),
                    L.thrust_cdna4_scan(t, ctypes.byref(nb), capi.I32, capi.PLUS, 0, None, None, 0, None, None),
                    L.thrust_cdna4_scan_by_key(t, ctypes.byref(nb), capi.I32, capi.I32, capi.PLUS, 0, None, None, None, 0, None, None)]
        assert calls(0x1000) == [0, 0, 0, 0]
        assert calls(0x1004) == [1, 1, 1, 1]
        rc = L.thrust_cdna4_reduce_by_key(ctypes.c_void_p(0x1004), ctypes.byref(nb), capi.I32, capi.I32, capi.PLUS,
                                          None, None, None, None, ctypes.c_void_p(0x2000), 0, None)
    elif bad == "bins":
        rc, _ = _size(L.thrust_cdna4_histogram_even, capi.U8, None, n, None, 0, 0.0, 1.0, None)
    else:
        rc, _ = _size(L.thrust_cdna4_histogram_even, capi.U8, None, n, None, 4, 1.0, 1.0, None)
    assert rc != 0
    assert capi.lib().thrust_cdna4_error_string(rc)


def test_scan_static_refuses_sizes_beyond_its_array_before_it_touches_a_device():
    L = capi.lib()
    for code, limit in [(capi.I32, 1 << 29), (capi.U8, 1 << 31), (capi.I16, 1 << 30), (capi.F32, 1 << 29),
                        (capi.I64, 1 << 28), (capi.F64, 1 << 28)]:
        assert L.thrust_cdna4_scan_static(code, capi.PLUS, 0, None, None, limit + 1, None, None) == 2
        assert L.thrust_cdna4_scan_static(code, capi.PLUS, 0, None, None, limit, None, None) == 1  # NULL ranges
    # minimum over 8-byte floating-point values publishes three words per tile (the fold restarts at
    # NaNs, which a tile has to say): the array holds descriptors for 10922 tiles of 16384 elements
    limit = 10922 * 16384
    assert L.thrust_cdna4_scan_static(capi.F64, capi.MINIMUM, 0, None, None, limit + 1, None, None) == 2
    assert L.thrust_cdna4_scan_static(capi.F64, capi.MINIMUM, 0, None, None, limit, None, None) == 1
    assert L.thrust_cdna4_scan_static(capi.F32, capi.MINIMUM, 0, None, None, (1 << 29) + 1, None, None) == 2
    assert L.thrust_cdna4_scan_static(capi.F32, capi.MINIMUM, 0, None, None, 1 << 29, None, None) == 1
    assert L.thrust_cdna4_scan_static(99, capi.PLUS, 0, None, None, 5, None, None) == 1
    assert L.thrust_cdna4_scan_static(capi.I32, 99, 0, None, None, 5, None, None) == 1
    assert L.thrust_cdna4_scan_static(capi.I32, capi.PLUS, 0, None, None, -1, None, None) == 1


def test_error_type_carries_the_code():
    with pytest.raises(capi.Cdna4Error) as ei:
        capi.check(1, "probe")
    assert ei.value.code == 1


def test_no_cpu_fallback_in_the_harness():
    import numpy as np
    import torch

    import thrust_amd
    with pytest.raises(ValueError):
        thrust_amd.sort(torch.from_numpy(np.arange(4, dtype=np.int32)))
