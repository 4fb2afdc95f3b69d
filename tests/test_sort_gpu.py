"""GPU parity of thrust_cdna4_sort_keys / sort_pairs against the oracle (bit-exact)."""
import numpy as np
import pytest
import torch

import oracle
import thrust_amd
from conftest import (FLOAT_DTYPES, INT_DTYPES, SIZES, SMALL_SIZES, encoded, random_floats, random_ints,
                      same_bits, splitmix64)
import gpu_util
from gpu_util import dev, host

pytestmark = pytest.mark.gpu


def test_sort_keys_kat(kat):
    for case in kat["sort_keys"]:
        for dt in case["dtypes"]:
            d = dev(np.array(case["keys"], dtype=dt))
            thrust_amd.sort(d, case["descending"])
            assert host(d).tolist() == case["expected"], (case["source"], dt)


def test_sort_pairs_kat(kat):
    for case in kat["sort_pairs"]:
        for kd in case["key_dtypes"]:
            for vd in case["value_dtypes"]:
                k = dev(np.array(case["keys"], dtype=kd))
                v = dev(np.array(case["values"], dtype=vd))
                thrust_amd.sort_by_key(k, v, case["descending"])
                assert host(k).tolist() == case["expected_keys"], (case["source"], kd, vd)
                assert host(v).tolist() == case["expected_values"], (case["source"], kd, vd)


@pytest.mark.parametrize("descending", [False, True])
def test_sort_u32_size_ladder(descending):
    for n in SIZES:
        k = random_ints(100 + n, n, np.uint32)
        d = dev(k)
        thrust_amd.sort(d, descending)
        assert same_bits(host(d), oracle.sort_keys(k, descending)), n


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_sort_int_keys_all_types(dtype):
    for n in [0, 1, 63, 257, 4096, 4097, 12345, 131072 + 5]:
        for descending in (False, True):
            k = random_ints(3 + n, n, dtype)
            d = dev(k)
            thrust_amd.sort(d, descending)
            assert same_bits(host(d), oracle.sort_keys(k, descending)), (n, descending)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_sort_float_keys_total_order(dtype):
    # -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN, as the reference's CPP system sorts
    tiny = np.finfo(dtype).tiny
    ordered = np.array([-np.nan, -np.inf, -1.5, -tiny / 4, -0.0, 0.0, tiny / 4, 1.5, np.inf, np.nan],
                       dtype=dtype)
    perm = np.random.default_rng(3).permutation(len(ordered))
    d = dev(ordered[perm])
    thrust_amd.sort(d)
    assert same_bits(host(d), ordered)
    for n in [100, 4099, 200003]:
        for descending in (False, True):
            k = random_floats(n, n, dtype)
            d = dev(k)
            thrust_amd.sort(d, descending)
            assert same_bits(host(d), oracle.sort_keys(k, descending)), (n, descending)


def test_sort_variable_bits():
    # keys with only the low `bits` bits set (testing/sort_variable_bits.cu:17-43)
    n = 20011
    for bits in range(0, 33, 3):
        mask = np.uint32((1 << bits) - 1) if bits < 32 else np.uint32(0xFFFFFFFF)
        k = random_ints(bits, n, np.uint32) & mask
        d = dev(k)
        thrust_amd.sort(d)
        assert same_bits(host(d), np.sort(k)), bits


@pytest.mark.parametrize("kd,vd", [(np.uint64, np.uint32), (np.uint32, np.uint32), (np.int32, np.uint64),
                                   (np.int8, np.uint16), (np.uint16, np.uint8), (np.float32, np.uint32),
                                   (np.float64, np.uint64), (np.int64, np.uint8)])
def test_sort_pairs_stability(kd, vd):
    for n in SMALL_SIZES[::3] + [262144 + 7]:
        for descending in (False, True):
            if np.dtype(kd).kind == "f":
                k = (np.random.default_rng(n).integers(-20, 20, n) / 4).astype(kd)
            else:
                k = (splitmix64(n, n) % np.uint64(41)).astype(kd)  # many duplicates
            v = np.arange(n).astype(vd)
            dk, dv = dev(k), dev(v)
            thrust_amd.sort_by_key(dk, dv, descending)
            rk, rv = oracle.sort_pairs(k, v, descending)
            assert same_bits(host(dk), rk) and same_bits(host(dv), rv), (n, descending)


def test_sort_pairs_u64_entropy_sweep():
    # benchmark configuration 3 at reduced n: keys = AND of k uniform words; values = original index
    n = (1 << 20) + 17
    for words in range(0, 5):
        k = np.full(n, np.uint64(0xFFFFFFFFFFFFFFFF))
        for w in range(words):
            k &= splitmix64(1000 + w, n)
        if words == 0:
            k[:] = np.uint64(42)  # all-equal keys
        v = np.arange(n, dtype=np.uint32)
        dk, dv = dev(k), dev(v)
        thrust_amd.sort_by_key(dk, dv)
        rk, rv = oracle.sort_pairs(k, v)
        assert same_bits(host(dk), rk) and same_bits(host(dv), rv), words


def test_sort_unaligned_views_and_repeat_determinism():
    k = random_ints(77, 100001, np.uint32)
    base = dev(k)
    view = base[3:]  # 12-byte offset: not 16-byte aligned
    thrust_amd.sort(view)
    assert same_bits(host(view), np.sort(k[3:]))
    assert same_bits(host(base[:3]), k[:3])
    # look-back bugs show up as run-to-run differences
    k = random_ints(78, 1 << 21, np.uint64)
    v = np.arange(k.size, dtype=np.uint32)
    first = None
    for _ in range(5):
        dk, dv = dev(k), dev(v)
        thrust_amd.sort_by_key(dk, dv)
        got = (host(dk).tobytes(), host(dv).tobytes())
        first = first or got
        assert got == first


@pytest.mark.needs_device
def test_sort_full_size_properties():
    # 2^28 u32 keys: sortedness + multiset preserved (checksums), no oracle at this size
    n = 1 << 28
    g = torch.Generator(device=gpu_util.DEVICE).manual_seed(1337)
    k = torch.randint(-2**31, 2**31, (n,), dtype=torch.int32, device=gpu_util.DEVICE, generator=g)
    s0 = k.sum(dtype=torch.int64).item()
    x0 = 0
    for chunk in k.view(16, -1):
        x0 ^= int(np.bitwise_xor.reduce(chunk.cpu().numpy().view(np.uint32)))
    u = k.view(torch.uint32) if hasattr(torch, "uint32") else k
    thrust_amd.sort(u)
    hk = k.cpu().numpy().view(np.uint32)
    assert (hk[1:] >= hk[:-1]).all()
    assert int(hk.view(np.int32).sum(dtype=np.int64)) == s0
    assert int(np.bitwise_xor.reduce(hk)) == x0


@pytest.mark.needs_device
def test_lds_atomic_order_selftest():
    """The stable ranking of the sort kernels assumes that returning LDS atomics of one wavefront
    instruction are served in lane order; the library's self-test checks that on this device."""
    import ctypes

    from thrust_amd import capi
    L = capi.lib()
    bad = ctypes.c_longlong(-1)
    rc = L.thrust_cdna4_selftest_lds_atomic_order(ctypes.byref(bad), gpu_util.stream_handle())
    assert rc == 0
    assert bad.value == 0


@pytest.mark.needs_device
def test_xcd_dispatch_selftest_and_both_tile_assignments():
    """Large sorts hand consecutive tiles to one XCD in groups (its L2 then merges the run ends that
    two tiles write into one cache line) on a device that passes the library's dispatch probe; MI355X
    does.  Both forms of the tile assignment — grouped, and one counter in index order — must give the
    oracle's result, for keys and pairs, at sizes with partial last groups."""
    import ctypes

    from thrust_amd import capi
    L = capi.lib()
    gpu_util.synchronize()
    verdicts = []
    for _ in range(3):  # 1: the device qualifies; 0 / -1 / -2: why not (the probe times workgroups: it is conservative under load)
        grouped = ctypes.c_int(-9)
        rc = L.thrust_cdna4_selftest_xcd_dispatch(ctypes.byref(grouped), gpu_util.stream_handle())
        assert rc == 0
        verdicts.append(grouped.value)
    print("xcd dispatch probe:", verdicts)
    assert 1 in verdicts, verdicts
    before = ctypes.c_ulonglong(0)
    L.thrust_cdna4_lookback_timeouts(ctypes.byref(before))
    for plain in (0, 1):
        prev = L.thrust_cdna4_set_test_sort_plain_tickets(plain)
        try:
            for n in [(1 << 23) + 1, 256 * 32768, 257 * 32768 + 5, (1 << 24) - 3]:
                k = random_ints(n, n, np.uint32)
                d = dev(k)
                thrust_amd.sort(d)
                assert same_bits(host(d), oracle.sort_keys(k)), (plain, n)
                k64 = random_ints(n + 1, n // 2, np.uint64) & np.uint64(0xFFFFFF)
                v = np.arange(n // 2, dtype=np.uint32)
                dk, dv = dev(k64), dev(v)
                thrust_amd.sort_by_key(dk, dv, descending=True)
                ek, ev = oracle.sort_pairs(k64, v, descending=True)
                assert same_bits(host(dk), ek) and same_bits(host(dv), ev), (plain, n)
            if plain == 0:
                # the leg above really ran the grouped form: the library's own cached verdict
                # (its probe is repeated when it rests on timing alone) says so
                form = ctypes.c_int(-1)
                assert L.thrust_cdna4_sort_tile_assignment(ctypes.byref(form)) == 0
                assert form.value == 1, form.value
        finally:
            L.thrust_cdna4_set_test_sort_plain_tickets(prev)
    after = ctypes.c_ulonglong(0)
    L.thrust_cdna4_lookback_timeouts(ctypes.byref(after))
    assert after.value == before.value


def test_sort_skewed_digits_stability():
    """Keys whose digits are heavily skewed (most lanes of a wavefront share a digit) take the
    careful ranking loop; pairs must stay stable."""
    rng = np.random.default_rng(99)
    n = 300_001
    for hot_frac in (0.3, 0.9, 1.0):
        keys = np.where(rng.random(n) < hot_frac, np.uint32(0x07070707), rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32))
        vals = np.arange(n, dtype=np.uint32)
        ek, ev = oracle.sort_pairs(keys.copy(), vals.copy(), False)
        k, v = dev(keys), dev(vals)
        thrust_amd.sort_by_key(k, v, False)
        assert same_bits(host(k), ek) and same_bits(host(v), ev), hot_frac


@pytest.mark.parametrize("dtype", INT_DTYPES + FLOAT_DTYPES)
def test_sort_keys_large_tiles_all_types(dtype):
    """Inputs of 2^21 keys and more run the large-tile kernels (smaller ones the 512 x 16 tiles);
    every key type goes through them here, with a ragged last tile."""
    n = (1 << 21) + 1234
    for descending in (False, True):
        k = random_floats(n, n, dtype) if np.dtype(dtype).kind == "f" else random_ints(11 + n, n, dtype)
        d = dev(k)
        thrust_amd.sort(d, descending)
        assert same_bits(host(d), oracle.sort_keys(k, descending)), descending


@pytest.mark.parametrize("kd,vd", [(np.uint64, np.uint32), (np.uint32, np.uint32), (np.int32, np.uint64),
                                   (np.int8, np.uint16), (np.uint16, np.uint8), (np.float32, np.uint32),
                                   (np.float64, np.uint64), (np.int64, np.uint8), (np.uint32, np.uint8)])
def test_sort_pairs_large_tiles_stability(kd, vd):
    """2^22 pairs and more run the large-tile kernels; duplicate-heavy keys check stability."""
    n = (1 << 22) + 77
    for descending, spread in ((False, 41), (True, 70001)):
        if np.dtype(kd).kind == "f":
            k = (np.random.default_rng(n).integers(-spread, spread, n) / 4).astype(kd)
        else:
            k = (splitmix64(n, n) % np.uint64(spread)).astype(kd)
        v = (np.arange(n) % (1 << (8 * np.dtype(vd).itemsize))).astype(vd) if np.dtype(vd).itemsize < 4 else np.arange(n).astype(vd)
        dk, dv = dev(k), dev(v)
        thrust_amd.sort_by_key(dk, dv, descending)
        rk, rv = oracle.sort_pairs(k, v, descending)
        assert same_bits(host(dk), rk) and same_bits(host(dv), rv), descending


@pytest.mark.needs_device
def test_sort_beyond_2p30_items():
    """n >= 2^30 switches the tile descriptors to 64-bit words (digit counts no longer fit 30
    bits).  No oracle at this size: sortedness, multiset checksums, and for pairs stability and
    key/value association, all checked on the device."""
    n = (1 << 30) + 12345
    g = torch.Generator(device=gpu_util.DEVICE).manual_seed(2030)
    k = torch.randint(-2**31, 2**31, (n,), dtype=torch.int32, device=gpu_util.DEVICE, generator=g)
    s0 = int(k.sum(dtype=torch.int64).item())
    thrust_amd.sort(k)
    assert bool((k[1:] >= k[:-1]).all())
    assert int(k.sum(dtype=torch.int64).item()) == s0
    del k
    gpu_util.empty_cache()
    # pairs: few distinct keys, so every digit count of the top passes exceeds 2^30 / 256 by far
    src = torch.randint(0, 1000, (n,), dtype=torch.int32, device=gpu_util.DEVICE, generator=g)
    k = src.clone()
    v = torch.arange(n, dtype=torch.int32, device=gpu_util.DEVICE)
    thrust_amd.sort_by_key(k, v)
    assert bool((k[1:] >= k[:-1]).all())
    assert bool(((k[1:] > k[:-1]) | (v[1:] > v[:-1])).all())  # equal keys keep their input order
    assert bool((src[v.long()] == k).all())
    del src, k, v
    gpu_util.empty_cache()
    # one-byte keys at the largest size the entry point takes (2^32 - 2): run starts near 2^32
    n = (1 << 32) - 2
    k = torch.randint(0, 4, (n,), dtype=torch.uint8, device=gpu_util.DEVICE, generator=g) * 85
    step = 1 << 30
    counts = sum(torch.bincount(k[a:a + step].to(torch.int32), minlength=256) for a in range(0, n, step))
    thrust_amd.sort(k, descending=True)
    for a in range(0, n, step):
        c = k[a:a + step]
        assert bool((c[1:] <= c[:-1]).all()) and (a == 0 or bool(k[a] <= k[a - 1]))
    assert torch.equal(counts, sum(torch.bincount(k[a:a + step].to(torch.int32), minlength=256) for a in range(0, n, step)))


# Places where every key has the same digit are skipped on the device (the identity for a stable
# sort), and the number of passes that run stays even so that the result ends in the caller's
# buffer.  Every pattern of constant and varying bytes must give the oracle's result, for keys and
# for pairs, in both tile configurations (n below and above the small-tile limit).
def _masked_keys(seed, n, dtype, vary_mask, constant):
    k = random_ints(seed, n, dtype).astype(dtype)
    u = k.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[k.dtype.itemsize])
    u &= u.dtype.type(vary_mask)
    u |= u.dtype.type(constant & ~vary_mask & (2 ** (8 * u.dtype.itemsize) - 1))
    return u.view(dtype)


@pytest.mark.parametrize("dtype,patterns", [
    (np.uint32, [(0x000000FF, 0), (0x0000FFFF, 0xAB000000), (0xFF00FFFF, 0x00CD0000), (0xFF000000, 0x00123456),
                 (0x00FFFF00, 0), (0x00000000, 0xDEADBEEF), (0x00FF0000, 0x11000022)]),
    (np.int32, [(0x000000FF, 0), (0x000000FF, 0xFFFFFF00), (0x800000FF, 0), (0x00FF00FF, 0x7F000000)]),
    (np.uint64, [(0x00000000000FFFFF, 0), (0x00000000FFFFFFFF, 0), (0xFFFF00000000FFFF, 0x0000ABCDEF000000),
                 (0x0000000000000000, 42), (0x00000000000000FF, 0x0100000000000000), (0xFF00FF00FF00FF00, 0x0011002200330044)]),
    (np.int64, [(0x00000000000FFFFF, 0), (0x80000000000000FF, 0), (0x00000000000000FF, 0xFFFFFFFFFFFFFF00)]),
    (np.uint16, [(0x00FF, 0x1200), (0xFF00, 0x0034), (0x0000, 0x5678)]),
    (np.float32, [(0x007FFFFF, 0x3F800000), (0x80000000, 0x3F800000), (0x000000FF, 0xBF800000)]),
])
def test_sort_skips_places_where_all_keys_agree(dtype, patterns):
    for n in [4097, 70001, (1 << 21) + 77, (1 << 22) + 5]:
        for vary, const in patterns:
            for descending in (False, True):
                k = _masked_keys(n + (vary & 0xFFFF), n, dtype, vary, const)
                d = dev(k)
                thrust_amd.sort(d, descending)
                assert same_bits(host(d), oracle.sort_keys(k, descending)), (n, hex(vary), hex(const), descending)
            # pairs: stability shows in the values
            k = _masked_keys(n + 1, n, dtype, vary, const)
            v = np.arange(n, dtype=np.uint32)
            dk, dv = dev(k), dev(v)
            thrust_amd.sort_by_key(dk, dv)
            ek, ev = oracle.sort_pairs(k, v)
            assert same_bits(host(dk), ek) and same_bits(host(dv), ev), (n, hex(vary), hex(const))


@pytest.mark.parametrize("dtype", [np.uint8, np.int8])
def test_sort_one_byte_keys_by_counting(dtype):
    """One-byte keys without values are written from their histogram (no key moves): all run shapes
    — uniform, few distinct values with empty bins between them, one value, the extreme values, ends
    of the input inside a 16-byte piece — at any alignment, both directions, against the oracle."""
    info = np.iinfo(dtype)
    for n in [4097, 4111, 70001, (1 << 21) + 77, (1 << 22) + 13]:
        rng = np.random.default_rng(n)
        cases = {
            "uniform": rng.integers(info.min, info.max + 1, n).astype(dtype),
            "three values": rng.choice(np.array([info.min, 7, info.max], dtype=dtype), n),
            "one value": np.full(n, info.max, dtype=dtype),
            "short runs at the ends": np.concatenate([np.full(n - 9, 5), np.arange(9) + info.min]).astype(dtype),
            "skewed": np.minimum(rng.geometric(0.3, n), info.max).astype(dtype),
        }
        for name, k in cases.items():
            for descending in (False, True):
                for shift in (0, 1, 7):
                    buf = torch.zeros(n + 32, dtype=torch.int8 if dtype == np.int8 else torch.uint8, device=gpu_util.DEVICE)
                    view = buf[shift:shift + n]
                    view.copy_(dev(k))
                    thrust_amd.sort(view, descending)
                    assert np.array_equal(host(view), oracle.sort_keys(k, descending)), (n, name, descending, shift)
                    assert int(buf[:shift].sum()) == 0 and int(buf[shift + n:].sum()) == 0, "wrote outside the range"
