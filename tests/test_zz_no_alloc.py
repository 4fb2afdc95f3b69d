"""thrust_cdna4_scan_static — the scan entry point that allocates nothing (its tile descriptors
live in a fixed array of the library's device image) — against thrust_cdna4_scan on the same
inputs, through the C ABI: integers bit-exact; floating-point sums within the scan tolerance
(1e-5 of the running L1 norm: the look-back may group the tiles differently from call to call)."""
import ctypes

import numpy as np
import pytest
import torch

import gpu_util

import thrust_amd
from thrust_amd import capi
from thrust_amd.api import _OPS, _init_box, _ptr, _stream, dtype_code
from conftest import random_ints

pytestmark = pytest.mark.gpu


def scan_static(x, op="plus", exclusive=False, init=None, out=None):
    L = capi.lib()
    if out is None:
        out = torch.empty_like(x)
    code = dtype_code(x)
    box, ip = _init_box(init, code)
    capi.check(L.thrust_cdna4_scan_static(code, _OPS[op], int(exclusive), _ptr(x), _ptr(out), x.numel(), ip,
                                          _stream()), "scan_static")
    return out


def reference_scan(x, op, exclusive, init):
    return thrust_amd.exclusive_scan(x, init=init, op=op) if exclusive else thrust_amd.inclusive_scan(x, op=op)


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.uint8, np.int16])
def test_two_calls_in_a_row_second_smaller(dtype):
    # the second call reuses the array the first one left its descriptors in
    for op, exclusive, init in [("plus", False, None), ("plus", True, 7), ("maximum", True, 3), ("multiplies", False, None)]:
        for n1, n2 in [((1 << 22) + 12345, 300_001), (200_003, 4097), (70_000, 1)]:
            a = gpu_util.dev(random_ints(n1 + 1, n1, dtype))
            b = gpu_util.dev(random_ints(n2 + 2, n2, dtype))
            got_a = scan_static(a, op, exclusive, init)
            got_b = scan_static(b, op, exclusive, init)
            assert torch.equal(got_a, reference_scan(a, op, exclusive, init)), (dtype, op, n1)
            assert torch.equal(got_b, reference_scan(b, op, exclusive, init)), (dtype, op, n2)


def test_float_and_in_place_and_large():
    g = torch.Generator(device=gpu_util.DEVICE).manual_seed(11)
    x = torch.rand((1 << 24) + 3, device=gpu_util.DEVICE, generator=g) * 2 - 1
    got = scan_static(x).double()
    ref = torch.cumsum(x.double(), 0)
    l1 = torch.cumsum(x.double().abs(), 0)
    assert bool(((got - ref).abs() <= 1e-5 * l1).all())
    y = torch.randint(0, 16, (1 << 26,), dtype=torch.int32, device=gpu_util.DEVICE, generator=g)
    want = thrust_amd.inclusive_scan(y)
    scan_static(y, out=y)  # in place: the ticket variant of the kernel
    assert torch.equal(y, want)
    small = torch.randint(0, 16, (50_001,), dtype=torch.int32, device=gpu_util.DEVICE, generator=g)
    assert torch.equal(scan_static(small, exclusive=True, init=5), thrust_amd.exclusive_scan(small, init=5))


def test_rejects_sizes_beyond_the_array_and_allocates_nothing():
    L = capi.lib()
    # One tile more than the array holds is refused with its own code before anything else is
    # looked at.  The calls pass NULL ranges, so nothing could be launched even if the size check
    # were wrong: they would then fail with code 1 instead of 2.
    for code, limit in [(capi.I32, 1 << 29), (capi.U8, 1 << 31), (capi.I16, 1 << 30), (capi.F32, 1 << 29),
                        (capi.I64, 1 << 28), (capi.F64, 1 << 28)]:
        assert L.thrust_cdna4_scan_static(code, capi.PLUS, 0, None, None, limit + 1, None, _stream()) == 2
        assert L.thrust_cdna4_scan_static(code, capi.PLUS, 0, None, None, limit, None, _stream()) == 1
    assert L.thrust_cdna4_scan_static(capi.I32, capi.PLUS, 0, None, None, 0, None, _stream()) == 0
    assert L.thrust_cdna4_scan_static(99, capi.PLUS, 0, None, None, 5, None, _stream()) == 1
    # the library's pool and torch's allocator are untouched by a call
    y = torch.randint(0, 16, (1 << 20,), dtype=torch.int32, device=gpu_util.DEVICE)
    out = torch.empty_like(y)
    gpu_util.synchronize()
    pool_before, torch_before = L.thrust_cdna4_pool_bytes(), gpu_util.memory_allocated()
    capi.check(L.thrust_cdna4_scan_static(capi.I32, capi.PLUS, 0, _ptr(y), _ptr(out), y.numel(), None, _stream()),
               "scan_static")
    gpu_util.synchronize()
    assert L.thrust_cdna4_pool_bytes() == pool_before and gpu_util.memory_allocated() == torch_before
    assert torch.equal(out, torch.cumsum(y, 0, dtype=torch.int32))
