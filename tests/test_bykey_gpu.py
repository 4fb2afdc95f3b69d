"""GPU parity of thrust_cdna4_scan_by_key and thrust_cdna4_reduce_by_key against the oracle."""
import numpy as np
import pytest
import torch

import oracle
import thrust_amd
from conftest import SMALL_SIZES, random_ints, same_bits
import gpu_util
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

FP_RTOL = 1e-5


def runs(seed, n, mean, kd=np.int32):
    """Sorted runs of keys with geometric run lengths (benchmark configuration 4)."""
    rng = np.random.default_rng(seed)
    if n == 0:
        return np.zeros(0, dtype=kd)
    if mean <= 1:
        return np.arange(n).astype(kd)
    lens = rng.geometric(1.0 / mean, max(8, int(2.5 * n / mean) + 8))
    keys = np.repeat(np.arange(lens.size), lens)
    while keys.size < n:
        keys = np.concatenate([keys, keys + keys[-1] + 1])
    return keys[:n].astype(kd)


# ------------------------------------------------------------------ scan_by_key
def test_scan_by_key_kat(kat):
    for case in kat["scan_by_key"]:
        for kd in [np.int32, np.uint8, np.int64, np.float32, np.int16]:
            for vd in [np.int32, np.int64, np.float32, np.uint16]:
                k = dev(np.array(case["keys"], dtype=kd))
                v = dev(np.array(case["values"], dtype=vd))
                if case["exclusive"]:
                    out = thrust_amd.exclusive_scan_by_key(k, v, init=case["init"], op=case["op"])
                else:
                    out = thrust_amd.inclusive_scan_by_key(k, v, op=case["op"])
                assert host(out).tolist() == case["expected"], (case["source"], kd, vd)


@pytest.mark.parametrize("kd,vd", [(np.int32, np.int32), (np.uint8, np.int64), (np.int64, np.uint16),
                                   (np.uint16, np.uint32), (np.float32, np.int32), (np.int32, np.int8)])
def test_scan_by_key_ints_bit_exact(kd, vd):
    for n in SMALL_SIZES[::2] + [300007]:
        for mean in (1, 3, 300):
            k = (runs(n + mean, n, mean, np.int64) % 120).astype(kd)
            v = random_ints(n, n, vd)
            dk, dv = dev(k), dev(v)
            assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv)), oracle.scan_by_key(k, v)), (n, mean)
            assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=10)),
                             oracle.scan_by_key(k, v, exclusive=True, init=10)), (n, mean)


def test_scan_by_key_ops_and_in_place():
    n = 50021
    k = runs(1, n, 5)
    v = random_ints(2, n, np.int32)
    for op in ["multiplies", "maximum", "minimum"]:
        dk, dv = dev(k), dev(v)
        thrust_amd.inclusive_scan_by_key(dk, dv, out=dv, op=op)
        assert same_bits(host(dv), oracle.scan_by_key(k, v, op)), op
        dv = dev(v)
        thrust_amd.exclusive_scan_by_key(dk, dv, out=dv, init=3, op=op)
        assert same_bits(host(dv), oracle.scan_by_key(k, v, op, exclusive=True, init=3)), op


def test_scan_by_key_float_tolerance():
    n = 1 << 20
    k = runs(3, n, 512)
    v = np.random.default_rng(4).standard_normal(n).astype(np.float32)
    got = host(thrust_amd.inclusive_scan_by_key(dev(k), dev(v))).astype(np.float64)
    # float64 segmented reference and the L1 norm of each segment prefix
    heads = np.ones(n, dtype=bool)
    heads[1:] = k[1:] != k[:-1]
    seg = np.cumsum(heads) - 1
    c = np.cumsum(v.astype(np.float64))
    a = np.cumsum(np.abs(v.astype(np.float64)))
    start = np.nonzero(heads)[0]
    ref = c - (c[start] - v[start].astype(np.float64))[seg]
    l1 = a - (a[start] - np.abs(v[start].astype(np.float64)))[seg]
    assert (np.abs(got - ref) <= FP_RTOL * l1 + 1e-30).all()
    serial = oracle.scan_by_key(k, v).astype(np.float64)
    assert (np.abs(got - serial) <= FP_RTOL * l1 + 1e-30).all()


# ------------------------------------------------------------------ reduce_by_key
def test_reduce_by_key_kat(kat):
    for case in kat["reduce_by_key"]:
        for kd in [np.int32, np.uint8, np.uint64, np.float64, np.int16]:
            for vd in [np.int32, np.int64, np.float32, np.uint8]:
                gk, gv = thrust_amd.reduce_by_key(dev(np.array(case["keys"], dtype=kd)),
                                                  dev(np.array(case["values"], dtype=vd)), op=case["op"])
                assert host(gk).tolist() == case["expected_keys"], (case["source"], kd, vd)
                assert host(gv).tolist() == case["expected_values"], (case["source"], kd, vd)


@pytest.mark.parametrize("kd,vd", [(np.int32, np.int32), (np.uint8, np.int64), (np.int64, np.uint16),
                                   (np.uint16, np.uint32), (np.int32, np.uint8), (np.uint64, np.int64)])
def test_reduce_by_key_ints_bit_exact(kd, vd):
    for n in SMALL_SIZES[::2] + [300007]:
        for mean in (1, 8, 512):
            k = (runs(n + mean, n, mean, np.int64) % 200).astype(kd)
            v = random_ints(n, n, vd)
            gk, gv = thrust_amd.reduce_by_key(dev(k), dev(v))
            rk, rv = oracle.reduce_by_key(k, v)
            assert same_bits(host(gk), rk) and same_bits(host(gv), rv), (n, mean)


def test_reduce_by_key_config4_reduced():
    # benchmark configuration 4 at 2^21: int32 values in [-1000,1000] bit-exact; fp32 N(0,1) within
    # 1e-5 of the run's L1 norm
    n = 1 << 21
    rng = np.random.default_rng(7)
    for mean in (1, 8, 512):
        k = runs(mean, n, mean)
        vi = rng.integers(-1000, 1001, n).astype(np.int32)
        gk, gv = thrust_amd.reduce_by_key(dev(k), dev(vi))
        rk, rv = oracle.reduce_by_key(k, vi)
        assert same_bits(host(gk), rk) and same_bits(host(gv), rv), mean
        vf = rng.standard_normal(n).astype(np.float32)
        gk, gv = thrust_amd.reduce_by_key(dev(k), dev(vf))
        rk, rv = oracle.reduce_by_key(k, vf)
        assert same_bits(host(gk), rk)
        starts = np.nonzero(np.concatenate([[True], k[1:] != k[:-1]]))[0]
        ref = np.add.reduceat(vf.astype(np.float64), starts)
        l1 = np.add.reduceat(np.abs(vf.astype(np.float64)), starts)
        assert (np.abs(host(gv).astype(np.float64) - ref) <= FP_RTOL * l1 + 1e-30).all(), mean
        assert (np.abs(host(gv).astype(np.float64) - rv.astype(np.float64)) <= FP_RTOL * l1 + 1e-30).all()


def test_reduce_by_key_ops_and_float_keys():
    n = 40009
    k = runs(11, n, 6)
    v = random_ints(12, n, np.int32)
    for op in ["maximum", "minimum", "multiplies"]:
        gk, gv = thrust_amd.reduce_by_key(dev(k), dev(v), op=op)
        rk, rv = oracle.reduce_by_key(k, v, op)
        assert same_bits(host(gk), rk) and same_bits(host(gv), rv), op
    keys = np.array([0.0, -0.0, 1.0, np.nan, np.nan, 2.0, 2.0], dtype=np.float32)
    vals = np.arange(7, dtype=np.int32)
    gk, gv = thrust_amd.reduce_by_key(dev(keys), dev(vals))
    rk, rv = oracle.reduce_by_key(keys, vals)
    assert same_bits(host(gk), rk) and host(gv).tolist() == [1, 2, 3, 4, 11]


@pytest.mark.needs_device
def test_reduce_by_key_empty_and_full_size_closed_form():
    gk, gv = thrust_amd.reduce_by_key(torch.empty(0, dtype=torch.int32, device=gpu_util.DEVICE),
                                      torch.empty(0, dtype=torch.int32, device=gpu_util.DEVICE))
    assert gk.numel() == 0 and gv.numel() == 0
    # 2^28 elements, keys = i // 512, values = 1: every run sums to 512
    # (closed form, cf. testing/cuda/reduce_by_key.cu:339-400)
    n = 1 << 28
    keys = torch.arange(n, dtype=torch.int32, device=gpu_util.DEVICE) // 512
    vals = torch.ones(n, dtype=torch.int32, device=gpu_util.DEVICE)
    gk, gv = thrust_amd.reduce_by_key(keys, vals)
    assert gk.numel() == n // 512
    assert torch.equal(gk, torch.arange(n // 512, dtype=torch.int32, device=gpu_util.DEVICE))
    assert bool((gv == 512).all())


# ------------------------------------------------------------------ forward-progress path
@pytest.fixture
def no_patience():
    """Look-back never waits: every tile descriptor that is not there yet is recomputed from the
    input by the workgroup that needs it (the forward-progress path of the ticketless kernels)."""
    from thrust_amd import capi
    L = capi.lib()
    previous = L.thrust_cdna4_set_lookback_patience(0)
    yield
    L.thrust_cdna4_set_lookback_patience(previous)


@pytest.mark.parametrize("kd,vd", [(np.int32, np.int32), (np.uint8, np.int64), (np.float32, np.int32),
                                   (np.uint64, np.uint16)])
def test_by_key_recompute_path_matches_oracle(no_patience, kd, vd):
    for n in [1, 16384, 16385, 100_003, (1 << 21) + 77]:
        for mean in (1, 8, 5000):
            k = (runs(n + mean, n, mean, np.int64) % 200).astype(kd)
            v = random_ints(n + 1, n, vd)
            dk, dv = dev(k), dev(v)
            assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv)), oracle.scan_by_key(k, v)), (n, mean)
            assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=3)),
                             oracle.scan_by_key(k, v, exclusive=True, init=3)), (n, mean)
            gk, gv = thrust_amd.reduce_by_key(dk, dv)
            rk, rv = oracle.reduce_by_key(k, v)
            assert same_bits(host(gk), rk) and same_bits(host(gv), rv), (n, mean)


@pytest.fixture
def tile0_publishes_late():
    """Tile 0 sleeps ~10 ms (a bounded number of sleeps) before it publishes, so with patience 0
    every later tile finds its descriptor missing twice and uses its own recomputed aggregate."""
    from thrust_amd import capi
    L = capi.lib()
    previous = L.thrust_cdna4_set_test_publish_delay(3000)
    yield
    L.thrust_cdna4_set_test_publish_delay(previous)


@pytest.mark.parametrize("op", ["plus", "multiplies", "maximum", "minimum"])
def test_by_key_with_a_recomputed_tile0(no_patience, tile0_publishes_late, op):
    # init restarts at every segment head (sequential/scan_by_key.h:95-140); it is applied where
    # results are formed, never stored in a tile descriptor, so a recomputed tile 0 loses nothing
    for kd, vd, n in [(np.int32, np.int32, 100_003), (np.uint64, np.int64, 50_001), (np.uint8, np.uint16, 70_000)]:
        for mean in (1, 8, 40_000):
            k = (runs(n + mean, n, mean, np.int64) % 200).astype(kd)
            v = random_ints(n + 3, n, vd)
            dk, dv = dev(k), dev(v)
            assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=7, op=op)),
                             oracle.scan_by_key(k, v, op=op, exclusive=True, init=7)), (kd, vd, n, mean)
            assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv, op=op)),
                             oracle.scan_by_key(k, v, op=op)), (kd, vd, n, mean)
            gk, gv = thrust_amd.reduce_by_key(dk, dv, op=op)
            rk, rv = oracle.reduce_by_key(k, v, op=op)
            assert same_bits(host(gk), rk) and same_bits(host(gv), rv), (kd, vd, n, mean)


def test_by_key_aliased_outputs_take_the_ticket_path():
    n = (1 << 20) + 9
    k = (runs(5, n, 8, np.int64) % 200).astype(np.int32)
    v = random_ints(6, n, np.int32)
    dk, dv = dev(k), dev(v)
    thrust_amd.inclusive_scan_by_key(dk, dv, out=dv)  # in place on the values
    assert same_bits(host(dv), oracle.scan_by_key(k, v))
    dk, dv = dev(k), dev(v)
    gk, gv = thrust_amd.reduce_by_key(dk, dv, keys_out=dk, values_out=dv)  # compaction in place
    rk, rv = oracle.reduce_by_key(k, v)
    assert same_bits(host(gk), rk) and same_bits(host(gv), rv)


def test_outputs_written_over_the_keys():
    """testing/scan_by_key.inclusive.cu:325-334 scans into the key range.  A tile reads the key before
    its first element from memory, where the tile before it may have stored results already: the
    library reads the keys from a copy then.  Every element a run of its own is the case in which
    reduce_by_key's compaction writes exactly where the next tile looks."""
    n = 16384 * 5 + 77
    for mean in (1, 2, 40):
        k = (runs(7 + mean, n, mean, np.int64) % 200).astype(np.int32)
        v = (np.arange(n) % 10).astype(np.int32)
        dk, dv = dev(k), dev(v)
        thrust_amd.inclusive_scan_by_key(dk, dv, out=dk)
        assert same_bits(host(dk), oracle.scan_by_key(k, v)), mean
        assert same_bits(host(dv), v)
        dk, dv = dev(k), dev(v)
        thrust_amd.exclusive_scan_by_key(dk, dv, out=dk, init=3)
        assert same_bits(host(dk), oracle.scan_by_key(k, v, exclusive=True, init=3)), mean
        rk, rv = oracle.reduce_by_key(k, v)
        dk, dv = dev(k), dev(v)
        gk, gv = thrust_amd.reduce_by_key(dk, dv, keys_out=dk, values_out=dv)  # both in place
        assert same_bits(host(gk), rk) and same_bits(host(gv), rv), mean
        dk, dv, spare = dev(k), dev(v), dev(np.zeros(n, np.int32))
        gk, gv = thrust_amd.reduce_by_key(dk, dv, keys_out=spare, values_out=dk)  # the values over the keys
        assert same_bits(host(gk), rk) and same_bits(host(gv), rv), mean


def piecewise_keys(seed, n, kd):
    """Stretches of very different run lengths side by side: none (one long run), 1 in 1000, 1 in 10,
    just below and just above every second element, every element.  A wavefront of a tile handles
    its heads one way when they are few and another when they are many; both, and wavefronts with
    no head at all, meet inside one input."""
    rng = np.random.default_rng(seed)
    densities = [0.0, 0.001, 0.1, 0.47, 0.49, 0.6, 1.0, 0.0, 0.3]
    piece = -(-n // len(densities))
    head = np.concatenate([rng.random(piece) < d if d < 1.0 else np.ones(piece, bool) for d in densities])[:n]
    ids = np.cumsum(head)
    if np.dtype(kd).kind == "f":
        return ids.astype(kd)
    return (ids % 97).astype(kd)  # neighbours still differ at every head


@pytest.mark.parametrize("kd,vd", [(np.int32, np.int32), (np.int64, np.int32), (np.int32, np.int64),
                                   (np.uint8, np.uint16), (np.float32, np.float64), (np.uint16, np.int8)])
def test_by_key_mixed_run_lengths_match_oracle(kd, vd):
    for n in (9 * 40000 + 123, 9 * 2048 * 3):
        k = piecewise_keys(n, n, kd)
        is_fp = np.dtype(vd).kind == "f"
        v = (np.random.default_rng(n).integers(-50, 50, n)).astype(vd) if is_fp else random_ints(n + 1, n, vd)
        dk, dv = dev(k), dev(v)
        for op in ("plus", "maximum", "minimum"):
            ko, vo = thrust_amd.reduce_by_key(dk, dv, op=op)
            rk, rv = oracle.reduce_by_key(k, v, op=op)
            assert same_bits(host(ko), rk), (n, op)
            assert same_bits(host(vo), rv), (n, op)  # small integers: exact in floating point too
            assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv, op=op)), oracle.scan_by_key(k, v, op=op)), (n, op)
        assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=3)),
                         oracle.scan_by_key(k, v, exclusive=True, init=3)), n


@pytest.mark.parametrize("op", ["maximum", "minimum"])
@pytest.mark.parametrize("vd", [np.float32, np.float64])
def test_float_extrema_by_key_with_nans_are_the_serial_fold(vd, op):
    """thrust::maximum is a < b ? b : a: in the serial folds (thrust/system/detail/sequential/
    scan_by_key.h:46-142, reduce_by_key.h:43-95) a NaN at the head of a segment stays for the whole
    segment, a NaN inside one is skipped, and the exclusive form — whose folds start from `init` —
    skips every NaN unless `init` is one.  thrust::minimum is a < b ? a : b: its folds restart at
    every NaN.  Same bits from the kernels, over several tiles, +0 / -0 ties and NaN payloads included."""
    rng = np.random.default_rng(21)
    for n in (1, 2, 9, 2049, 16385, 50021, 200003):
        for mean in (1, 3, 300):
            k = runs(n + mean, n, mean)
            head = np.ones(n, bool)
            head[1:] = k[1:] != k[:-1]
            for where in ("none", "heads", "inside", "both", "all"):
                v = rng.uniform(-5, 5, n).astype(vd)
                v[rng.random(n) < 0.05] = vd(-np.inf)
                v[rng.random(n) < 0.05] = vd(np.inf)
                v[rng.random(n) < 0.04] = vd(0.0)
                v[rng.random(n) < 0.04] = vd(-0.0)
                if where in ("heads", "both"):
                    v[head & (rng.random(n) < 0.5)] = np.nan
                if where in ("inside", "both"):
                    v[~head & (rng.random(n) < 0.3)] = np.nan
                if where == "all":
                    v[:] = np.nan
                nan = np.isnan(v)
                u = v.view(np.uint32 if vd == np.float32 else np.uint64)
                u[nan] ^= (rng.integers(0, 1 << 20, int(nan.sum())).astype(u.dtype)
                           | (rng.integers(0, 2, int(nan.sum())).astype(u.dtype) << u.dtype.type(u.dtype.itemsize * 8 - 1)))
                dk, dv = dev(k), dev(v)
                assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv, op=op)),
                                 oracle.scan_by_key(k, v, op=op)), (n, mean, where)
                for init in (vd(1.5), vd(np.nan)):
                    assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=init, op=op)),
                                     oracle.scan_by_key(k, v, op=op, exclusive=True, init=init)), (n, mean, where, init)
                ko, vo = thrust_amd.reduce_by_key(dk, dv, op=op)
                ek, ev = oracle.reduce_by_key(k, v, op=op)
                assert same_bits(host(ko), ek) and same_bits(host(vo), ev), (n, mean, where)
                y = dev(v)
                thrust_amd.inclusive_scan_by_key(dk, y, out=y, op=op)  # in place: tiles by ticket
                assert same_bits(host(y), oracle.scan_by_key(k, v, op=op)), (n, mean, where, "in place")


@pytest.mark.parametrize("op", ["maximum", "minimum"])
def test_float_extrema_by_key_with_nans_on_the_recompute_path(no_patience, tile0_publishes_late, op):
    rng = np.random.default_rng(22)
    n = 16384 * 3 + 5
    for mean in (1, 40):
        k = runs(n + mean, n, mean)
        v = rng.uniform(-5, 5, n).astype(np.float32)
        v[rng.random(n) < 0.3] = np.nan
        dk, dv = dev(k), dev(v)
        assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv, op=op)), oracle.scan_by_key(k, v, op=op)), mean
        assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=np.float32(0.25), op=op)),
                         oracle.scan_by_key(k, v, op=op, exclusive=True, init=np.float32(0.25))), mean
        ko, vo = thrust_amd.reduce_by_key(dk, dv, op=op)
        ek, ev = oracle.reduce_by_key(k, v, op=op)
        assert same_bits(host(ko), ek) and same_bits(host(vo), ev), mean


@pytest.mark.parametrize("op", ["maximum", "minimum"])
@pytest.mark.parametrize("vd", [np.float32, np.float64])
def test_float_extrema_by_key_keep_the_zero_the_serial_fold_keeps(vd, op):
    """Values that are mostly +0 and -0: the SIGN of a result tells which operand the fold kept
    (maximum the first of equals, minimum the last).  Long runs, so that the value of a run crosses
    threads, wavefronts and tiles before it meets its last element."""
    rng = np.random.default_rng(41)
    for n in (9, 2049, 50021, 200003):
        for mean in (3, 300, 40000):
            k = runs(n + mean, n, mean)
            v = np.where(rng.random(n) < 0.5, vd(0.0), vd(-0.0)).astype(vd)
            losers = rng.random(n) < 0.3
            v[losers] = (-1 if op == "maximum" else 1) * rng.uniform(1, 5, int(losers.sum())).astype(vd)
            dk, dv = dev(k), dev(v)
            assert same_bits(host(thrust_amd.inclusive_scan_by_key(dk, dv, op=op)), oracle.scan_by_key(k, v, op=op)), (n, mean)
            for init in (vd(0.0), vd(-0.0), vd(-7.0), vd(7.0)):
                assert same_bits(host(thrust_amd.exclusive_scan_by_key(dk, dv, init=init, op=op)),
                                 oracle.scan_by_key(k, v, op=op, exclusive=True, init=init)), (n, mean, init)
            ko, vo = thrust_amd.reduce_by_key(dk, dv, op=op)
            ek, ev = oracle.reduce_by_key(k, v, op=op)
            assert same_bits(host(ko), ek) and same_bits(host(vo), ev), (n, mean)
            y = dev(v)
            thrust_amd.exclusive_scan_by_key(dk, y, out=y, init=vd(-0.0), op=op)  # in place: tiles by ticket
            assert same_bits(host(y), oracle.scan_by_key(k, v, op=op, exclusive=True, init=vd(-0.0))), (n, mean, "in place")
