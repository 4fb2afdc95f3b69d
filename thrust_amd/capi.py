"""ctypes binding of libthrust_cdna4.so (the C ABI declared in include/thrust_cdna4.h).

There is no fallback: if the HIP library has not been built, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# THRUST_CDNA4_LIB points the harness at another build of the same C ABI (tuning builds).
LIB_PATH = os.environ.get("THRUST_CDNA4_LIB") or os.path.join(_HERE, "lib", "libthrust_cdna4.so")

I8, U8, I16, U16, I32, U32, I64, U64, F32, F64 = range(10)
PLUS, MULTIPLIES, MAXIMUM, MINIMUM = range(4)

# every symbol include/thrust_cdna4.h declares
SYMBOLS = [
    "thrust_cdna4_abi_version", "thrust_cdna4_error_string", "thrust_cdna4_sort_keys",
    "thrust_cdna4_sort_pairs", "thrust_cdna4_scan", "thrust_cdna4_scan_by_key",
    "thrust_cdna4_reduce_by_key", "thrust_cdna4_histogram_even", "thrust_cdna4_malloc",
    "thrust_cdna4_free", "thrust_cdna4_pool_trim", "thrust_cdna4_pool_bytes",
    "thrust_cdna4_memcpy_htod", "thrust_cdna4_memcpy_dtoh", "thrust_cdna4_memcpy_dtod", "thrust_cdna4_read_back",
    "thrust_cdna4_fill", "thrust_cdna4_stream_synchronize", "thrust_cdna4_profile_enable",
    "thrust_cdna4_profile_count", "thrust_cdna4_profile_get",
    "thrust_cdna4_selftest_lds_atomic_order", "thrust_cdna4_set_lookback_patience",
    "thrust_cdna4_set_test_publish_delay", "thrust_cdna4_scan_static",
    "thrust_cdna4_lookback_timeouts",
    "thrust_cdna4_stream_create", "thrust_cdna4_stream_destroy", "thrust_cdna4_stream_query",
    "thrust_cdna4_event_create", "thrust_cdna4_event_destroy", "thrust_cdna4_event_record", "thrust_cdna4_event_query",
    "thrust_cdna4_stream_wait_event", "thrust_cdna4_malloc_direct", "thrust_cdna4_free_direct",
    "thrust_cdna4_malloc_universal", "thrust_cdna4_free_universal", "thrust_cdna4_get_device",
    "thrust_cdna4_selftest_xcd_dispatch", "thrust_cdna4_set_test_sort_plain_tickets",
    "thrust_cdna4_sort_status", "thrust_cdna4_set_test_sort_spin_limit", "thrust_cdna4_sort_tile_assignment",
    "thrust_cdna4_lookback_timeout_counter",
]


class Cdna4Error(RuntimeError):
    """A C-ABI entry point returned a non-zero hipError_t."""

    def __init__(self, code, what, text):
        super().__init__(f"{what}: hip error {code} ({text})")
        self.code = code


_lib = None


def bind(path):
    """Load a build of the C ABI from `path` and declare every entry point's argument types."""
    L = ctypes.CDLL(path)
    vp, sz, i32, i64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int64
    psz = ctypes.POINTER(ctypes.c_size_t)
    dbl = ctypes.c_double
    L.thrust_cdna4_abi_version.restype = i32
    L.thrust_cdna4_error_string.restype = ctypes.c_char_p
    L.thrust_cdna4_error_string.argtypes = [i32]
    L.thrust_cdna4_sort_keys.argtypes = [vp, psz, i32, vp, i64, i32, vp]
    L.thrust_cdna4_sort_pairs.argtypes = [vp, psz, i32, vp, i32, vp, i64, i32, vp]
    L.thrust_cdna4_sort_status.argtypes = [vp, i64, vp]
    L.thrust_cdna4_set_test_sort_spin_limit.argtypes = [ctypes.c_longlong]
    L.thrust_cdna4_sort_tile_assignment.argtypes = [ctypes.POINTER(i32)]
    L.thrust_cdna4_lookback_timeout_counter.argtypes = [ctypes.POINTER(vp)]
    L.thrust_cdna4_scan.argtypes = [vp, psz, i32, i32, i32, vp, vp, i64, vp, vp]
    L.thrust_cdna4_scan_static.argtypes = [i32, i32, i32, vp, vp, i64, vp, vp]
    L.thrust_cdna4_scan_by_key.argtypes = [vp, psz, i32, i32, i32, i32, vp, vp, vp, i64, vp, vp]
    L.thrust_cdna4_reduce_by_key.argtypes = [vp, psz, i32, i32, i32, vp, vp, vp, vp, vp, i64, vp]
    L.thrust_cdna4_histogram_even.argtypes = [vp, psz, i32, vp, i64, vp, i32, dbl, dbl, vp]
    L.thrust_cdna4_malloc.argtypes = [ctypes.POINTER(vp), sz, vp]
    L.thrust_cdna4_free.argtypes = [vp, vp]
    L.thrust_cdna4_pool_bytes.restype = sz
    L.thrust_cdna4_memcpy_htod.argtypes = [vp, vp, sz, vp]
    L.thrust_cdna4_memcpy_dtoh.argtypes = [vp, vp, sz, vp]
    L.thrust_cdna4_read_back.argtypes = [vp, vp, sz, vp]
    L.thrust_cdna4_memcpy_dtod.argtypes = [vp, vp, sz, vp]
    L.thrust_cdna4_fill.argtypes = [vp, vp, i32, i64, vp]
    L.thrust_cdna4_stream_synchronize.argtypes = [vp]
    L.thrust_cdna4_stream_create.argtypes = [ctypes.POINTER(vp)]
    L.thrust_cdna4_stream_destroy.argtypes = [vp]
    L.thrust_cdna4_stream_query.argtypes = [vp, ctypes.POINTER(ctypes.c_int)]
    L.thrust_cdna4_event_create.argtypes = [ctypes.POINTER(vp)]
    L.thrust_cdna4_event_destroy.argtypes = [vp]
    L.thrust_cdna4_event_record.argtypes = [vp, vp]
    L.thrust_cdna4_event_query.argtypes = [vp, ctypes.POINTER(ctypes.c_int)]
    L.thrust_cdna4_stream_wait_event.argtypes = [vp, vp]
    L.thrust_cdna4_malloc_direct.argtypes = [ctypes.POINTER(vp), sz]
    L.thrust_cdna4_free_direct.argtypes = [vp]
    L.thrust_cdna4_malloc_universal.argtypes = [ctypes.POINTER(vp), sz, i32]
    L.thrust_cdna4_free_universal.argtypes = [vp, i32]
    L.thrust_cdna4_get_device.argtypes = [ctypes.POINTER(i32)]
    L.thrust_cdna4_set_lookback_patience.argtypes = [i32]
    L.thrust_cdna4_set_test_publish_delay.argtypes = [i32]
    L.thrust_cdna4_lookback_timeouts.argtypes = [ctypes.POINTER(ctypes.c_ulonglong)]
    L.thrust_cdna4_profile_enable.argtypes = [i32]
    L.thrust_cdna4_selftest_lds_atomic_order.argtypes = [ctypes.POINTER(ctypes.c_longlong), vp]
    L.thrust_cdna4_selftest_xcd_dispatch.argtypes = [ctypes.POINTER(i32), vp]
    L.thrust_cdna4_set_test_sort_plain_tickets.argtypes = [i32]
    L.thrust_cdna4_profile_get.argtypes = [i32, ctypes.POINTER(ctypes.c_char_p),
                                           ctypes.POINTER(ctypes.c_float)]
    return L


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C thrust_amd/csrc` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    _lib = bind(LIB_PATH)
    return _lib


def profile_records():
    """[(kernel name, milliseconds)] logged since thrust_cdna4_profile_enable(1)."""
    L = lib()
    out = []
    for i in range(L.thrust_cdna4_profile_count()):
        name = ctypes.c_char_p()
        ms = ctypes.c_float()
        check(L.thrust_cdna4_profile_get(i, ctypes.byref(name), ctypes.byref(ms)), "profile_get")
        out.append((name.value.decode(), ms.value))
    return out


def check(code, what):
    if code != 0:
        text = lib().thrust_cdna4_error_string(code).decode()
        raise Cdna4Error(code, what, text)
