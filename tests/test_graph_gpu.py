"""Every algorithm entry point of the C ABI captured into a HIP graph and replayed.

The entry points enqueue kernels only (what must start at zero is cleared by a fill kernel, never
by a memset node), take their temporary storage from the caller and touch no host state, so a
caller may capture them.  Each test captures one call, then replays the graph several times with
NEW input in the same buffers, with eager work and synchronisations between the replays, and checks
every replay against the eager result of the same call."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from thrust_amd import capi
from conftest import random_ints
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

N = 300_001  # several tiles for every algorithm
REPLAYS = 3


def sizes_then_capture(call):
    """call(temp_ptr, nbytes_box, stream_ptr): size query eagerly, warm-up eagerly, then capture."""
    L = capi.lib()
    side = torch.cuda.Stream()
    sp = ctypes.c_void_p(side.cuda_stream)
    nb = ctypes.c_size_t(0)
    capi.check(call(None, nb, sp), "size query")
    tmp = torch.empty(max(nb.value, 1), dtype=torch.uint8, device="cuda")
    tp = ctypes.c_void_p(tmp.data_ptr())
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        capi.check(call(tp, nb, sp), "warm-up")  # outside the capture: first-use set-up (module load, the sort's device check)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        capi.check(call(tp, nb, sp), "captured call")
    torch.cuda.synchronize()
    return g, tmp


def replay_and_check(g, refill, check):
    for r in range(REPLAYS):
        refill(r)                      # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        check(r)


@pytest.mark.parametrize("N", [300_001, (1 << 22) + 77])  # the small-input and the large-input configuration
def test_sort_keys_and_pairs_in_a_graph(N):
    L = capi.lib()
    k = torch.empty(N, dtype=torch.int32, device="cuda")
    g, tmp = sizes_then_capture(lambda t, nb, sp: L.thrust_cdna4_sort_keys(t, ctypes.byref(nb), capi.U32, ctypes.c_void_p(k.data_ptr()), N, 0, sp))
    data = [random_ints(40 + r, N, np.uint32) for r in range(REPLAYS)]
    replay_and_check(g, lambda r: k.copy_(dev(data[r].view(np.int32))),
                     lambda r: np.testing.assert_array_equal(host(k).view(np.uint32), oracle.sort_keys(data[r])))
    kk = torch.empty(N, dtype=torch.int64, device="cuda")
    vv = torch.empty(N, dtype=torch.int32, device="cuda")
    g2, tmp2 = sizes_then_capture(lambda t, nb, sp: L.thrust_cdna4_sort_pairs(
        t, ctypes.byref(nb), capi.U64, ctypes.c_void_p(kk.data_ptr()), 4, ctypes.c_void_p(vv.data_ptr()), N, 1, sp))
    keys = [random_ints(50 + r, N, np.uint64) & np.uint64(0xFFFF) for r in range(REPLAYS)]  # many ties, most places skipped
    vals = np.arange(N, dtype=np.uint32)

    def fill(r):
        kk.copy_(dev(keys[r].view(np.int64)))
        vv.copy_(dev(vals.view(np.int32)))

    def check(r):
        ek, ev = oracle.sort_pairs(keys[r], vals, descending=True)
        np.testing.assert_array_equal(host(kk).view(np.uint64), ek)
        np.testing.assert_array_equal(host(vv).view(np.uint32), ev)
    replay_and_check(g2, fill, check)


@pytest.mark.parametrize("in_place", [False, True])
def test_scan_in_a_graph(in_place):
    L = capi.lib()
    x = torch.empty(N, dtype=torch.int32, device="cuda")
    out = x if in_place else torch.empty_like(x)
    init = ctypes.c_int32(5)
    g, tmp = sizes_then_capture(lambda t, nb, sp: L.thrust_cdna4_scan(
        t, ctypes.byref(nb), capi.I32, capi.PLUS, 1, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()), N,
        ctypes.byref(init), sp))
    data = [random_ints(60 + r, N, np.int32) for r in range(REPLAYS)]
    replay_and_check(g, lambda r: x.copy_(dev(data[r])),
                     lambda r: np.testing.assert_array_equal(host(out), oracle.scan(data[r], "plus", True, 5)))


def test_scan_static_in_a_graph():
    L = capi.lib()
    x = torch.empty(N, dtype=torch.float32, device="cuda")
    out = torch.empty_like(x)
    side = torch.cuda.Stream()
    sp = ctypes.c_void_p(side.cuda_stream)
    call = lambda: L.thrust_cdna4_scan_static(capi.F32, capi.MAXIMUM, 0, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()), N, None, sp)
    with torch.cuda.stream(side):
        capi.check(call(), "warm-up")  # looks up the fixed array's address: outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        capi.check(call(), "captured")
    torch.cuda.synchronize()
    data = [np.random.default_rng(70 + r).standard_normal(N).astype(np.float32) for r in range(REPLAYS)]
    replay_and_check(g, lambda r: x.copy_(dev(data[r])),
                     lambda r: np.testing.assert_array_equal(host(out), np.maximum.accumulate(data[r])))


def test_by_key_algorithms_in_a_graph():
    L = capi.lib()
    keys = torch.empty(N, dtype=torch.int32, device="cuda")
    vals = torch.empty(N, dtype=torch.int32, device="cuda")
    out = torch.empty_like(vals)
    g, tmp = sizes_then_capture(lambda t, nb, sp: L.thrust_cdna4_scan_by_key(
        t, ctypes.byref(nb), capi.I32, capi.I32, capi.PLUS, 0, ctypes.c_void_p(keys.data_ptr()), ctypes.c_void_p(vals.data_ptr()),
        ctypes.c_void_p(out.data_ptr()), N, None, sp))
    ko = torch.empty_like(keys)
    vo = torch.empty_like(vals)
    nr = torch.zeros(1, dtype=torch.int64, device="cuda")
    g2, tmp2 = sizes_then_capture(lambda t, nb, sp: L.thrust_cdna4_reduce_by_key(
        t, ctypes.byref(nb), capi.I32, capi.I32, capi.PLUS, ctypes.c_void_p(keys.data_ptr()), ctypes.c_void_p(vals.data_ptr()),
        ctypes.c_void_p(ko.data_ptr()), ctypes.c_void_p(vo.data_ptr()), ctypes.c_void_p(nr.data_ptr()), N, sp))
    hk = [np.cumsum(np.random.default_rng(80 + r).random(N) < (0.5, 0.05, 0.9)[r], dtype=np.int32) for r in range(REPLAYS)]
    hv = [random_ints(90 + r, N, np.int32) for r in range(REPLAYS)]

    def fill(r):
        keys.copy_(dev(hk[r]))
        vals.copy_(dev(hv[r]))
        nr.zero_()

    def check_scan(r):
        np.testing.assert_array_equal(host(out), oracle.scan_by_key(hk[r], hv[r]))

    def check_reduce(r):
        ek, ev = oracle.reduce_by_key(hk[r], hv[r])
        runs = int(nr.item())
        assert runs == len(ek)
        np.testing.assert_array_equal(host(ko)[:runs], ek)
        np.testing.assert_array_equal(host(vo)[:runs], ev)
    replay_and_check(g, fill, check_scan)
    replay_and_check(g2, fill, check_reduce)


@pytest.mark.parametrize("bins", [256, 4096, 100000])
def test_histogram_in_a_graph(bins):
    L = capi.lib()
    s = torch.empty(N, dtype=torch.float32, device="cuda")
    counts = torch.empty(bins, dtype=torch.int32, device="cuda")
    g, tmp = sizes_then_capture(lambda t, nb, sp: L.thrust_cdna4_histogram_even(
        t, ctypes.byref(nb), capi.F32, ctypes.c_void_p(s.data_ptr()), N, ctypes.c_void_p(counts.data_ptr()), bins, 0.0, 1000.0, sp))
    data = [(np.random.default_rng(100 + r).random(N) * 1100 - 50).astype(np.float32) for r in range(REPLAYS)]
    replay_and_check(g, lambda r: s.copy_(dev(data[r])),
                     lambda r: np.testing.assert_array_equal(host(counts).view(np.uint32), oracle.histogram_even(data[r], bins, 0.0, 1000.0)))
