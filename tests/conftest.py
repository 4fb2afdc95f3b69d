import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# THRUST_CDNA4_EMULATED=1 runs the GPU parity tests WITHOUT a GPU: the C ABI is served by the host
# build of the same kernel sources under the lockstep emulator (tests/emu), "device" tensors are CPU
# tensors, and the harness's device checks are relaxed here, in the tests, never in the package.
# tests/test_emulated_kernels.py starts such sessions; nothing else sets the variable.
EMULATED = os.environ.get("THRUST_CDNA4_EMULATED") == "1"
EMU_LIB = os.path.join(ROOT, "tests", "emu", "build", "libthrust_cdna4_emu.so")
if EMULATED:
    os.environ["THRUST_CDNA4_LIB"] = EMU_LIB


def _enter_emulated_session():
    import ctypes

    import torch

    import gpu_util
    import thrust_amd.api as api

    def need_contiguous(*ts):
        for t in ts:
            if t is not None and not t.is_contiguous():
                raise ValueError("contiguous tensors required")

    api._need_cuda = need_contiguous
    api._stream = lambda: ctypes.c_void_p(0)
    # THRUST_CDNA4_EMULATED_RESIDENT="k" or "k:seed": workgroups in flight (default 1, one after the other)
    k, _, seed = os.environ.get("THRUST_CDNA4_EMULATED_RESIDENT", "1").partition(":")
    emu = ctypes.CDLL(EMU_LIB)
    emu.emu_set_resident_workgroups.argtypes = [ctypes.c_int, ctypes.c_uint64]
    emu.emu_set_resident_workgroups(int(k), int(seed or 1))
    gpu_util.DEVICE = "cpu"
    gpu_util.dev = lambda a: torch.from_numpy(np.array(a, copy=True, order="C"))
    if os.environ.get("THRUST_CDNA4_EMULATED_GUARD") == "1":
        _guard_device_memory(gpu_util, api, torch)
    gpu_util.host = lambda t: t.numpy().copy()
    gpu_util.stream_handle = lambda: ctypes.c_void_p(0)
    gpu_util.synchronize = lambda: None
    gpu_util.empty_cache = lambda: None
    gpu_util.memory_allocated = lambda: 0


def _guard_device_memory(gpu_util, api, torch):
    """THRUST_CDNA4_EMULATED_GUARD=1: every "device" buffer of the session — inputs, outputs, the
    temporary storage — ends exactly where an inaccessible page begins, and another one lies before
    the page it starts in.  A kernel that reads or writes one byte past the end of a range it was
    given ends the session with a segmentation fault in the test that made the call.  (The buffers
    are then aligned to their element size only, like a view that starts inside an allocation.)"""
    import ctypes
    import mmap
    import weakref

    libc = ctypes.CDLL(None, use_errno=True)
    libc.mmap.restype = ctypes.c_void_p
    libc.mmap.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_long]
    libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    libc.munmap.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    page = mmap.PAGESIZE

    def guarded(shape, dtype):
        dtype = np.dtype(dtype)
        nbytes = int(np.prod(shape, dtype=np.int64)) * dtype.itemsize
        body = max(page, -(-nbytes // page) * page)
        total = body + 2 * page
        base = libc.mmap(None, total, mmap.PROT_READ | mmap.PROT_WRITE, mmap.MAP_PRIVATE | mmap.MAP_ANONYMOUS, -1, 0)
        assert base not in (None, ctypes.c_void_p(-1).value), ctypes.get_errno()
        assert libc.mprotect(base, page, 0) == 0 and libc.mprotect(base + page + body, page, 0) == 0
        raw = (ctypes.c_char * max(nbytes, 1)).from_address(base + page + body - max(nbytes, 1))
        a = np.frombuffer(raw, dtype=dtype, count=int(np.prod(shape, dtype=np.int64))).reshape(shape)
        weakref.finalize(raw, libc.munmap, base, total)  # the array keeps `raw` alive
        return a

    def dev(a):
        a = np.asarray(a)
        g = guarded(a.shape, a.dtype)
        g[...] = a
        return torch.from_numpy(g)

    np_of = {torch.int8: np.int8, torch.uint8: np.uint8, torch.int16: np.int16, torch.int32: np.int32, torch.int64: np.int64,
             torch.float32: np.float32, torch.float64: np.float64, torch.bool: np.bool_}
    for name in ("uint16", "uint32", "uint64"):
        if hasattr(torch, name):
            np_of[getattr(torch, name)] = getattr(np, name)

    class GuardedTorch:
        """the allocations of thrust_amd.api, guarded; everything else is torch"""
        def __getattr__(self, name):
            return getattr(torch, name)

        @staticmethod
        def empty(size, dtype=torch.float32, device=None):
            return torch.from_numpy(guarded((int(size),) if np.isscalar(size) else tuple(size), np_of[dtype]))

        @staticmethod
        def zeros(size, dtype=torch.float32, device=None):
            t = GuardedTorch.empty(size, dtype)
            t.zero_()
            return t

        @staticmethod
        def empty_like(t):
            return torch.from_numpy(guarded(tuple(t.shape), np_of[t.dtype]))

    gpu_util.dev = dev
    api.torch = GuardedTorch()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "needs_device: a gpu test that the emulated session cannot run")
    if EMULATED:
        _enter_emulated_session()


def pytest_collection_modifyitems(config, items):
    if not EMULATED:
        return
    skip = pytest.mark.skip(reason="needs the device itself (full-size input, graphs, streams, timing)")
    for item in items:
        if "needs_device" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def kat():
    with open(os.path.join(ROOT, "tests", "golden", "kat.json")) as f:
        return json.load(f)


# Size ladder of the reference's variable-size tests (testing/unittest/testframework.cu:21-31),
# cut at 2^20+1 so the oracle finishes in seconds.
SIZES = [0, 1, 2, 3, 4, 5, 8, 10, 13, 16, 17, 19, 27, 30, 31, 32, 33, 35, 42, 53, 58, 63, 64, 65,
         72, 97, 100, 127, 128, 129, 142, 183, 192, 201, 240, 255, 256, 257, 302, 511, 512, 513,
         687, 900, 1023, 1024, 1025, 1565, 1786, 1973, 2047, 2048, 2049, 3050, 4095, 4096, 4097,
         5030, 7791, 10000, 10027, 12345, 16384, 17354, 26255, 32768, 43718, 65533, 65536, 65539,
         123456, 131072, 731588, 1048575, 1048576, 1048577]
SMALL_SIZES = [s for s in SIZES if s <= 70000]

INT_DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]
FLOAT_DTYPES = [np.float32, np.float64]
ALL_DTYPES = INT_DTYPES + FLOAT_DTYPES


def splitmix64(seed, n, offset=0):
    """Counter-based generator: element i depends only on (seed, i)."""
    with np.errstate(over="ignore"):
        z = (np.arange(offset, offset + n, dtype=np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = z + np.uint64(seed)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def random_ints(seed, n, dtype):
    """Uniform over the full range of an integer dtype."""
    bits = splitmix64(seed, n)
    return bits.astype(np.dtype(dtype).str.replace("i", "u")).view(dtype) if np.dtype(dtype).kind == "i" \
        else bits.astype(dtype)


def random_floats(seed, n, dtype, specials=True):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(n).astype(dtype)
    if specials and n >= 16:
        tiny = np.finfo(dtype).tiny
        sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, -np.nan, tiny / 4, -tiny / 4], dtype=dtype)
        x[rng.choice(n, 8, replace=False)] = sp
    return x


def encoded(keys):
    """Unsigned key whose natural order is the reference's radix order
    (thrust/system/detail/sequential/stable_radix_sort.inl:43-139)."""
    keys = np.ascontiguousarray(keys)
    w = keys.dtype.itemsize * 8
    u = keys.view(f"u{keys.dtype.itemsize}")
    sign = np.array(1 << (w - 1), dtype=u.dtype)
    if keys.dtype.kind == "u":
        return u.copy()
    if keys.dtype.kind == "i":
        return u ^ sign
    ones = np.array((1 << w) - 1, dtype=u.dtype)
    return u ^ np.where(u >> np.array(w - 1, dtype=u.dtype), ones, sign).astype(u.dtype)


def same_bits(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.dtype == b.dtype and a.shape == b.shape and a.tobytes() == b.tobytes()
