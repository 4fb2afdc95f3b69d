"""Temporary storage arrives dirty: a caller hands over whatever its allocator gives, and a pool
hands back what the previous call left there (thrust/system/cuda/detail/sort.h:330-365 takes its
storage from `temporary_array`, which initialises nothing).  Every entry point must bring the
words it relies on — status, histograms, tickets, tile descriptors — to zero itself.  Here the
storage is filled with ones, and then with a pattern that reads as "complete, large count" in
every descriptor format, before each call through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from conftest import random_ints, same_bits
import gpu_util
from gpu_util import dev, host
from thrust_amd import capi

pytestmark = pytest.mark.gpu

FILLS = [0xFF, 0xA5]


def _run(entry, fill, *args):
    """Size query, storage filled with `fill`, the call itself."""
    L = capi.lib()
    fn = getattr(L, entry)
    nb = ctypes.c_size_t(0)
    assert fn(None, ctypes.byref(nb), *args) == 0
    tmp = torch.full((max(nb.value, 1),), fill, dtype=torch.uint8, device=gpu_util.DEVICE)
    assert fn(ctypes.c_void_p(tmp.data_ptr()), ctypes.byref(nb), *args) == 0
    gpu_util.synchronize()
    return tmp


def p(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("fill", FILLS)
@pytest.mark.parametrize("n", [5000, 70001, (1 << 21) + 4097])
def test_sort_from_dirty_storage(n, fill):
    sp = gpu_util.stream_handle()
    k = random_ints(n + fill, n, np.uint32)
    d = dev(k)
    tmp = _run("thrust_cdna4_sort_keys", fill, capi.U32, p(d), n, 0, sp)
    assert same_bits(host(d), oracle.sort_keys(k))
    assert capi.lib().thrust_cdna4_sort_status(p(tmp), n, sp) == 0  # the status word was cleared too
    k64 = random_ints(n, n, np.uint64) & np.uint64(0xFFFFFF)  # some digit places are skipped
    v = np.arange(n, dtype=np.uint32)
    dk, dv = dev(k64), dev(v)
    _run("thrust_cdna4_sort_pairs", fill, capi.U64, p(dk), 4, p(dv), n, 1, sp)
    rk, rv = oracle.sort_pairs(k64, v, descending=True)
    assert same_bits(host(dk), rk) and same_bits(host(dv), rv)
    b = random_ints(n + 1, n, np.uint8)  # one-byte keys alone: histogram and fill
    db = dev(b)
    _run("thrust_cdna4_sort_keys", fill, capi.U8, p(db), n, 0, sp)
    assert same_bits(host(db), oracle.sort_keys(b))


@pytest.mark.parametrize("fill", FILLS)
@pytest.mark.parametrize("n", [40000, 300007])
def test_scan_and_by_key_from_dirty_storage(n, fill):
    sp = gpu_util.stream_handle()
    x = random_ints(n, n, np.int32)
    dx, out = dev(x), dev(np.zeros(n, dtype=np.int32))
    _run("thrust_cdna4_scan", fill, capi.I32, capi.PLUS, 0, p(dx), p(out), n, None, sp)
    assert same_bits(host(out), oracle.scan(x))
    _run("thrust_cdna4_scan", fill, capi.I32, capi.PLUS, 0, p(dx), p(dx), n, None, sp)  # in place: tickets
    assert same_bits(host(dx), oracle.scan(x))
    f = (random_ints(n + 3, n, np.int32) % 1000).astype(np.float64)
    f[::97] = np.nan
    df, fo = dev(f), dev(np.zeros(n, dtype=np.float64))
    _run("thrust_cdna4_scan", fill, capi.F64, capi.MINIMUM, 0, p(df), p(fo), n, None, sp)
    assert same_bits(host(fo), oracle.scan(f, op="minimum"))

    rng = np.random.default_rng(n + fill)
    keys = np.repeat(np.arange(n), rng.geometric(1 / 8, n))[:n].astype(np.int32)
    vals = random_ints(n + 7, n, np.int32)
    dk, dv, do = dev(keys), dev(vals), dev(np.zeros(n, dtype=np.int32))
    _run("thrust_cdna4_scan_by_key", fill, capi.I32, capi.I32, capi.PLUS, 0, p(dk), p(dv), p(do), n, None, sp)
    assert same_bits(host(do), oracle.scan_by_key(keys, vals))
    ko, vo = dev(np.zeros(n, dtype=np.int32)), dev(np.zeros(n, dtype=np.int32))
    nr = dev(np.full(1, -1, dtype=np.int64))
    _run("thrust_cdna4_reduce_by_key", fill, capi.I32, capi.I32, capi.PLUS, p(dk), p(dv), p(ko), p(vo), p(nr), n, sp)
    rk, rv = oracle.reduce_by_key(keys, vals)
    r = int(host(nr)[0])
    assert r == rk.size and same_bits(host(ko)[:r], rk) and same_bits(host(vo)[:r], rv)
