"""A sort whose look-back gives up must say so (thrust/system/cuda/detail/util.h:207-292: the
reference turns every runtime failure of a synchronous algorithm into thrust::system_error).

The wait is made to fail from the host, without hanging anything: the poll limit of the sort's
look-back is set to 0 and tile 0 of every pass publishes its digit counts late, so the tiles that
look for them give up at once.  Every kernel still runs to completion.

This file sorts after tests/test_sort_gpu.py on purpose: after a time-out the library hands tiles
out from a single counter for the rest of the process, which the tile-assignment test there would
notice."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
import thrust_amd
from conftest import random_ints, same_bits
import gpu_util
from gpu_util import dev, host
from thrust_amd import capi

pytestmark = pytest.mark.gpu

HIP_ERROR_LAUNCH_TIMEOUT = 702


def _timeouts(L):
    c = ctypes.c_ulonglong(0)
    assert L.thrust_cdna4_lookback_timeouts(ctypes.byref(c)) == 0
    return c.value


def test_a_sort_whose_lookback_gives_up_reports_it_and_later_sorts_are_right():
    L = capi.lib()
    n = 3 << 20  # 96 tiles of 32768 keys
    k = random_ints(5, n, np.uint32)
    # a sort outside the experiment first: module load, the device checks of the first sort
    d = dev(k)
    thrust_amd.sort(d)
    assert same_bits(host(d), oracle.sort_keys(k))
    before = _timeouts(L)

    prev_plain = L.thrust_cdna4_set_test_sort_plain_tickets(1)
    prev_limit = L.thrust_cdna4_set_test_sort_spin_limit(0)
    prev_delay = L.thrust_cdna4_set_test_publish_delay(200)
    try:
        # through the Python mirror of thrust::sort(thrust::device, ...): the call throws
        d = dev(k)
        with pytest.raises(capi.Cdna4Error) as err:
            thrust_amd.sort(d)
        assert err.value.code == HIP_ERROR_LAUNCH_TIMEOUT
        # and through the C ABI: the launch itself succeeds, the status call reports the time-out
        d = dev(k)
        v = dev(np.arange(n, dtype=np.uint32))
        sp = gpu_util.stream_handle()
        nb = ctypes.c_size_t(0)
        args = (capi.U32, ctypes.c_void_p(d.data_ptr()), 4, ctypes.c_void_p(v.data_ptr()), n, 0, sp)
        assert L.thrust_cdna4_sort_pairs(None, ctypes.byref(nb), *args) == 0
        tmp = torch.empty(nb.value, dtype=torch.uint8, device=gpu_util.DEVICE)
        assert L.thrust_cdna4_sort_pairs(ctypes.c_void_p(tmp.data_ptr()), ctypes.byref(nb), *args) == 0
        assert L.thrust_cdna4_sort_status(ctypes.c_void_p(tmp.data_ptr()), n, sp) == HIP_ERROR_LAUNCH_TIMEOUT
    finally:
        L.thrust_cdna4_set_test_publish_delay(prev_delay)
        L.thrust_cdna4_set_test_sort_spin_limit(prev_limit)
        L.thrust_cdna4_set_test_sort_plain_tickets(prev_plain)
    assert _timeouts(L) > before
    # the device is now latched to the single counter, and sorts are right again
    form = ctypes.c_int(-1)
    assert L.thrust_cdna4_sort_tile_assignment(ctypes.byref(form)) == 0 and form.value == 2
    for m in (n, (1 << 23) + 77):
        kk = random_ints(m, m, np.uint32)
        d = dev(kk)
        thrust_amd.sort(d)
        assert same_bits(host(d), oracle.sort_keys(kk)), m


def test_small_and_one_byte_sorts_have_nothing_to_report():
    L = capi.lib()
    sp = gpu_util.stream_handle()
    # up to 4096 items nothing of the temporary storage is used, not even its status word
    assert L.thrust_cdna4_sort_status(None, 4096, sp) == 0
    garbage = torch.full((4096,), 0xFF, dtype=torch.uint8, device=gpu_util.DEVICE)
    assert L.thrust_cdna4_sort_status(ctypes.c_void_p(garbage.data_ptr()), 100, sp) == 0
    k = random_ints(1, 1 << 20, np.uint8)
    d = dev(k)
    thrust_amd.sort(d)  # one-byte keys: histogram and fill, the status word is cleared and stays clear
    assert same_bits(host(d), oracle.sort_keys(k))
