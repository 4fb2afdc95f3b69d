"""GPU checks of the runtime entry points of the C ABI: the caching pool, direct allocation,
copies and fills, and the streams and events behind the asynchronous algorithms."""
import ctypes

import numpy as np
import pytest
import torch

from thrust_amd import capi

pytestmark = pytest.mark.gpu
vp = ctypes.c_void_p


def test_pool_reuses_blocks_and_trims():
    L = capi.lib()
    s = vp(torch.cuda.current_stream().cuda_stream)
    p = vp()
    capi.check(L.thrust_cdna4_malloc(ctypes.byref(p), 1 << 20, s), "malloc")
    first = p.value
    assert first and first % 256 == 0
    capi.check(L.thrust_cdna4_free(p, s), "free")
    q = vp()
    capi.check(L.thrust_cdna4_malloc(ctypes.byref(q), (1 << 20) - 100, s), "malloc")
    assert q.value == first  # same size class, same stream: handed back without a driver call
    assert L.thrust_cdna4_pool_bytes() >= 1 << 20
    capi.check(L.thrust_cdna4_free(q, s), "free")
    capi.check(L.thrust_cdna4_stream_synchronize(s), "sync")
    capi.check(L.thrust_cdna4_pool_trim(), "trim")
    zero = vp()
    capi.check(L.thrust_cdna4_malloc(ctypes.byref(zero), 0, s), "malloc(0)")
    capi.check(L.thrust_cdna4_free(zero, s), "free")


def test_pool_size_classes_round_up_by_an_eighth_at_most_above_1MiB():
    L = capi.lib()
    s = vp(torch.cuda.current_stream().cuda_stream)
    capi.check(L.thrust_cdna4_stream_synchronize(s), "sync")
    capi.check(L.thrust_cdna4_pool_trim(), "trim")
    base = L.thrust_cdna4_pool_bytes()
    want = (1 << 30) + (21 << 20)  # the temporary storage of a 2^28-key sort: 1.02 GiB
    p = vp()
    capi.check(L.thrust_cdna4_malloc(ctypes.byref(p), want, s), "malloc")
    held = L.thrust_cdna4_pool_bytes() - base
    assert want <= held <= want + want // 8, held
    capi.check(L.thrust_cdna4_free(p, s), "free")
    q = vp()
    capi.check(L.thrust_cdna4_malloc(ctypes.byref(q), want - (10 << 20), s), "malloc")  # same class: 1 GiB < x <= 1.125 GiB
    assert q.value == p.value
    capi.check(L.thrust_cdna4_free(q, s), "free")
    # below 1 MiB classes are powers of two
    small = vp()
    capi.check(L.thrust_cdna4_malloc(ctypes.byref(small), 3000, s), "malloc")
    assert L.thrust_cdna4_pool_bytes() - base - held == 4096
    capi.check(L.thrust_cdna4_free(small, s), "free")
    capi.check(L.thrust_cdna4_stream_synchronize(s), "sync")
    capi.check(L.thrust_cdna4_pool_trim(), "trim")
    assert L.thrust_cdna4_pool_bytes() == base


def test_direct_allocation_copy_and_fill_roundtrip():
    L = capi.lib()
    n = 100_003
    p = vp()
    capi.check(L.thrust_cdna4_malloc_direct(ctypes.byref(p), 4 * n), "malloc_direct")
    assert p.value
    src = np.arange(n, dtype=np.int32)
    back = np.empty_like(src)
    capi.check(L.thrust_cdna4_memcpy_htod(p, src.ctypes.data_as(vp), 4 * n, None), "htod")
    capi.check(L.thrust_cdna4_memcpy_dtoh(back.ctypes.data_as(vp), p, 4 * n, None), "dtoh")
    capi.check(L.thrust_cdna4_stream_synchronize(None), "sync")
    assert (back == src).all()
    pattern = ctypes.c_int32(-7)
    capi.check(L.thrust_cdna4_fill(p, ctypes.byref(pattern), 4, n, None), "fill")
    capi.check(L.thrust_cdna4_memcpy_dtoh(back.ctypes.data_as(vp), p, 4 * n, None), "dtoh")
    capi.check(L.thrust_cdna4_stream_synchronize(None), "sync")
    assert (back == -7).all()
    capi.check(L.thrust_cdna4_free_direct(p), "free_direct")
    capi.check(L.thrust_cdna4_free_direct(None), "free_direct(NULL)")


def test_streams_and_events_order_work_across_streams():
    L = capi.lib()
    s1, s2, ev = vp(), vp(), vp()
    capi.check(L.thrust_cdna4_stream_create(ctypes.byref(s1)), "stream")
    capi.check(L.thrust_cdna4_stream_create(ctypes.byref(s2)), "stream")
    capi.check(L.thrust_cdna4_event_create(ctypes.byref(ev)), "event")
    n = 1 << 22
    keys = torch.randint(-2**31, 2**31, (n,), dtype=torch.int32, device="cuda")
    expect = np.sort(keys.cpu().numpy().view(np.uint32))
    out = torch.empty_like(keys)
    torch.cuda.synchronize()
    # sort on s1, then copy the result on s2 after an event recorded behind the sort
    nb = ctypes.c_size_t(0)
    kp = vp(keys.data_ptr())
    capi.check(L.thrust_cdna4_sort_keys(None, ctypes.byref(nb), capi.U32, kp, n, 0, s1), "size")
    tmp = torch.empty(nb.value, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    capi.check(L.thrust_cdna4_sort_keys(vp(tmp.data_ptr()), ctypes.byref(nb), capi.U32, kp, n, 0, s1), "sort")
    capi.check(L.thrust_cdna4_event_record(ev, s1), "record")
    capi.check(L.thrust_cdna4_stream_wait_event(s2, ev), "wait_event")
    capi.check(L.thrust_cdna4_memcpy_dtod(vp(out.data_ptr()), kp, 4 * n, s2), "dtod")
    capi.check(L.thrust_cdna4_stream_synchronize(s2), "sync")
    done = ctypes.c_int(-1)
    capi.check(L.thrust_cdna4_event_query(ev, ctypes.byref(done)), "event_query")
    assert done.value == 1  # s2 waited for it
    capi.check(L.thrust_cdna4_stream_query(s2, ctypes.byref(done)), "stream_query")
    assert done.value == 1
    assert (out.cpu().numpy().view(np.uint32) == expect).all()
    capi.check(L.thrust_cdna4_event_destroy(ev), "event_destroy")
    capi.check(L.thrust_cdna4_stream_destroy(s1), "stream_destroy")
    capi.check(L.thrust_cdna4_stream_destroy(s2), "stream_destroy")
    assert L.thrust_cdna4_stream_destroy(None) != 0  # the default stream is not ours to destroy
    assert L.thrust_cdna4_event_record(None, None) != 0


def test_read_back_waits_for_the_stream_and_handles_every_size():
    """Small results go through the thread's pinned buffer, larger ones straight to the
    destination; either way the bytes are there when the call returns, also when the producing
    work was only just enqueued on another stream, and from a second host thread."""
    import threading

    L = capi.lib()
    side = torch.cuda.Stream()
    for nbytes in (1, 8, 4096, 4097, 1 << 20):
        with torch.cuda.stream(side):
            src = torch.arange(nbytes, device="cuda", dtype=torch.int64).to(torch.uint8)  # enqueued, not waited for
            dst = np.zeros(nbytes, dtype=np.uint8)
            capi.check(L.thrust_cdna4_read_back(vp(dst.ctypes.data), vp(src.data_ptr()), nbytes, vp(side.cuda_stream)),
                       "read_back")
        assert np.array_equal(dst, np.arange(nbytes, dtype=np.int64).astype(np.uint8)), nbytes
    capi.check(L.thrust_cdna4_read_back(None, None, 0, None), "read_back of nothing")
    assert L.thrust_cdna4_read_back(None, None, 8, None) != 0

    src = torch.full((16,), 7, device="cuda", dtype=torch.int32)
    torch.cuda.synchronize()
    got = {}

    def worker(i):
        out = np.zeros(16, dtype=np.int32)
        rc = L.thrust_cdna4_read_back(vp(out.ctypes.data), vp(src.data_ptr()), 64, None)
        got[i] = (rc, out.copy())

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert all(rc == 0 and (out == 7).all() for rc, out in got.values()) and len(got) == 4
