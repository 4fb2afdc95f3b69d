"""Pins the CPU oracle (oracle/oracle.c) before anything is compared against it:
the reference's own known-answer vectors, independent library routines (numpy's sorts,
cumsum, bincount), closed forms and brute force on small inputs."""
import numpy as np
import pytest

import oracle
from conftest import (ALL_DTYPES, FLOAT_DTYPES, INT_DTYPES, encoded, random_floats, random_ints,
                      same_bits, splitmix64)


# ------------------------------------------------------------------ sort
def test_sort_keys_kat(kat):
    for case in kat["sort_keys"]:
        for dt in case["dtypes"]:
            got = oracle.sort_keys(np.array(case["keys"], dtype=dt), case["descending"])
            assert got.tolist() == case["expected"], (case["source"], dt)


def test_sort_pairs_kat(kat):
    for case in kat["sort_pairs"]:
        for kd in case["key_dtypes"]:
            for vd in case["value_dtypes"]:
                k, v = oracle.sort_pairs(np.array(case["keys"], dtype=kd),
                                         np.array(case["values"], dtype=vd), case["descending"])
                assert k.tolist() == case["expected_keys"], (case["source"], kd, vd)
                assert v.tolist() == case["expected_values"], (case["source"], kd, vd)


@pytest.mark.parametrize("dtype", INT_DTYPES)
@pytest.mark.parametrize("n", [0, 1, 2, 255, 1000, 70001])
def test_sort_int_keys_match_numpy(dtype, n):
    k = random_ints(7 + n, n, dtype)
    assert same_bits(oracle.sort_keys(k), np.sort(k))
    assert same_bits(oracle.sort_keys(k, True), np.sort(k)[::-1])


def test_float_total_order_known_vector():
    # The reference's CPP system orders floats by bit pattern:
    # -NaN < -inf < negatives < -0 < +0 < positives < +inf < +NaN.
    for dt in FLOAT_DTYPES:
        tiny = np.finfo(dt).tiny
        ordered = np.array([-np.nan, -np.inf, -1.5, -tiny / 4, -0.0, 0.0, tiny / 4, 1.5, np.inf, np.nan],
                           dtype=dt)
        # make sure the NaNs really carry the signs we mean
        u = ordered.view(f"u{ordered.itemsize}")
        assert (u[0] >> (8 * ordered.itemsize - 1)) == 1 and (u[-1] >> (8 * ordered.itemsize - 1)) == 0
        perm = np.random.default_rng(3).permutation(len(ordered))
        assert same_bits(oracle.sort_keys(ordered[perm]), ordered)
        assert same_bits(oracle.sort_keys(ordered[perm], True), ordered[::-1])


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_sort_float_keys_match_numpy_on_encoded(dtype):
    k = random_floats(11, 50000, dtype)
    order = np.argsort(encoded(k), kind="stable")
    assert same_bits(oracle.sort_keys(k), k[order])


@pytest.mark.parametrize("kd", [np.uint8, np.int16, np.uint32, np.int64, np.uint64, np.float32])
@pytest.mark.parametrize("vd", [np.uint8, np.uint16, np.uint32, np.uint64])
def test_sort_pairs_stable_vs_numpy(kd, vd):
    n = 30000
    if np.dtype(kd).kind == "f":
        k = (np.random.default_rng(5).integers(-20, 20, n) / 4).astype(kd)
    else:
        k = (splitmix64(5, n) % np.uint64(37)).astype(kd)
    v = np.arange(n).astype(vd)  # wraps for narrow value types; still a valid payload
    idx = np.arange(n)
    order = np.argsort(encoded(k), kind="stable")
    gk, gv = oracle.sort_pairs(k, v)
    assert same_bits(gk, k[order]) and same_bits(gv, v[order])
    # descending: larger keys first, equal keys in input order
    inv = ~encoded(k)
    order_d = np.argsort(inv, kind="stable")
    gk, gv = oracle.sort_pairs(k, v, True)
    assert same_bits(gk, k[order_d]) and same_bits(gv, v[order_d])
    assert idx[order_d].shape == (n,)


def test_sort_brute_force_tiny():
    rng = np.random.default_rng(9)
    for _ in range(200):
        n = int(rng.integers(0, 9))
        k = rng.integers(0, 4, n).astype(np.int32)
        v = np.arange(n, dtype=np.uint32)
        pairs = sorted(zip(k.tolist(), v.tolist()), key=lambda p: p[0])  # Python's sort is stable
        gk, gv = oracle.sort_pairs(k, v)
        assert list(zip(gk.tolist(), gv.tolist())) == pairs


def test_config1_plumbing_sort_2_25_u32_seed_1337():
    # benchmark configuration 1: 2^25 uniform u32 keys, seed 1337, ascending == std::sort order.
    k = splitmix64(1337, 1 << 25).astype(np.uint32)
    got = oracle.sort_keys(k)
    assert same_bits(got, np.sort(k))
    k2 = k.copy()
    oracle.omp_sort(k2)
    assert same_bits(k2, got)


@pytest.mark.parametrize("dtype", [np.uint32, np.int32, np.uint64, np.int64])
@pytest.mark.parametrize("threads", [1, 3, 8])
def test_omp_sort_matches_serial(dtype, threads):
    n = 100003
    k = random_ints(21, n, dtype)
    k[::7] = k[0]
    v = np.arange(n, dtype=np.uint32)
    rk, rv = oracle.sort_pairs(k, v)
    kk, vv = k.copy(), v.copy()
    oracle.omp_sort(kk, vv, threads)
    assert same_bits(kk, rk) and same_bits(vv, rv)


# ------------------------------------------------------------------ scan
def test_scan_kat(kat):
    for case in kat["scan"]:
        for dt in [np.int8, np.int16, np.int32, np.int64, np.float32, np.float64]:
            got = oracle.scan(np.array(case["input"], dtype=dt), case["op"], case["exclusive"], case["init"])
            assert got.tolist() == case["expected"], (case["source"], dt)
            got = oracle.scan(np.array(case["input"], dtype=dt), case["op"], case["exclusive"],
                              case["init"], inplace=True)
            assert got.tolist() == case["expected"], (case["source"], dt, "in place")


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_scan_ints_match_cumsum_with_wraparound(dtype):
    x = random_ints(31, 10007, dtype)
    with np.errstate(over="ignore"):
        incl = np.cumsum(x, dtype=dtype)
    assert same_bits(oracle.scan(x), incl)
    excl = np.empty_like(x)
    init = np.array(5, dtype=dtype)
    with np.errstate(over="ignore"):
        excl[0] = init
        excl[1:] = (incl[:-1] + init).astype(dtype)
    assert same_bits(oracle.scan(x, exclusive=True, init=5), excl)


def test_scan_closed_forms():
    n = 100000
    ones = np.ones(n, dtype=np.int64)
    assert (oracle.scan(ones) == np.arange(1, n + 1)).all()
    assert (oracle.scan(ones, exclusive=True, init=0) == np.arange(n)).all()
    x = random_ints(33, n, np.int32)
    assert same_bits(oracle.scan(x, "maximum"), np.maximum.accumulate(x))
    assert same_bits(oracle.scan(x, "minimum"), np.minimum.accumulate(x))
    # inclusive[i] - exclusive[i] == x[i] (integers, wraparound arithmetic)
    with np.errstate(over="ignore"):
        assert same_bits((oracle.scan(x) - oracle.scan(x, exclusive=True, init=0)).astype(np.int32), x)


def test_scan_float_is_the_serial_left_fold():
    x = np.random.default_rng(35).uniform(-1, 1, 5000).astype(np.float32)
    acc = np.float32(0)
    ref = np.empty_like(x)
    for i, v in enumerate(x):
        acc = np.float32(acc + v) if i else v
        ref[i] = acc
    assert same_bits(oracle.scan(x), ref)


# ------------------------------------------------------------------ scan_by_key
def test_scan_by_key_kat(kat):
    for case in kat["scan_by_key"]:
        for kd in [np.int32, np.uint8, np.int64, np.float32]:
            for vd in [np.int32, np.int64, np.float32, np.uint16]:
                got = oracle.scan_by_key(np.array(case["keys"], dtype=kd), np.array(case["values"], dtype=vd),
                                         case["op"], case["exclusive"], case["init"])
                assert got.tolist() == case["expected"], (case["source"], kd, vd)


def _segments(keys):
    heads = np.ones(len(keys), dtype=bool)
    heads[1:] = keys[1:] != keys[:-1]
    starts = np.nonzero(heads)[0]
    return starts, np.append(starts[1:], len(keys))


def test_scan_by_key_brute_force():
    rng = np.random.default_rng(41)
    n = 20000
    keys = np.repeat(rng.integers(0, 1000, n), rng.integers(1, 9, n))[:n].astype(np.int32)
    vals = rng.integers(-100, 100, n).astype(np.int64)
    incl = oracle.scan_by_key(keys, vals)
    excl = oracle.scan_by_key(keys, vals, exclusive=True, init=7)
    for s, e in zip(*_segments(keys)):
        c = np.cumsum(vals[s:e])
        assert (incl[s:e] == c).all()
        assert excl[s] == 7 and (excl[s + 1:e] == 7 + c[:-1]).all()


# ------------------------------------------------------------------ reduce_by_key
def test_reduce_by_key_kat(kat):
    for case in kat["reduce_by_key"]:
        for kd in [np.int32, np.uint8, np.uint64, np.float64]:
            for vd in [np.int32, np.int64, np.float32, np.uint8]:
                gk, gv = oracle.reduce_by_key(np.array(case["keys"], dtype=kd),
                                              np.array(case["values"], dtype=vd), case["op"])
                assert gk.tolist() == case["expected_keys"], (case["source"], kd, vd)
                assert gv.tolist() == case["expected_values"], (case["source"], kd, vd)


def test_reduce_by_key_brute_force_and_invariants():
    rng = np.random.default_rng(43)
    n = 50000
    keys = np.repeat(rng.integers(0, 50, n), rng.geometric(1 / 8, n))[:n].astype(np.int32)
    vals = rng.integers(-1000, 1001, n).astype(np.int32)
    gk, gv = oracle.reduce_by_key(keys, vals)
    starts, ends = _segments(keys)
    assert len(gk) == len(starts) == 1 + int((keys[1:] != keys[:-1]).sum())
    assert (gk == keys[starts]).all()
    assert (gv == np.add.reduceat(vals, starts)).all()
    gk, gv = oracle.reduce_by_key(keys, vals, "maximum")
    assert (gv == np.maximum.reduceat(vals, starts)).all()
    assert oracle.reduce_by_key(keys[:0], vals[:0])[0].size == 0


def test_reduce_by_key_float_keys_use_numeric_equality():
    keys = np.array([0.0, -0.0, 1.0, np.nan, np.nan, 2.0, 2.0], dtype=np.float32)
    vals = np.arange(7, dtype=np.int32)
    gk, gv = oracle.reduce_by_key(keys, vals)
    # -0 == +0 (one run, first key kept); NaN != NaN (two runs)
    assert gv.tolist() == [1, 2, 3, 4, 11]
    assert same_bits(gk[:1], np.array([0.0], dtype=np.float32))


# ------------------------------------------------------------------ histogram
def test_histogram_kat(kat):
    case = kat["histogram"][0]
    for dt in ALL_DTYPES:
        s = np.array(case["samples"], dtype=dt)
        got = oracle.histogram_even(s, case["num_bins"], case["lower"], case["upper"])
        assert got.tolist() == case["expected"], dt
        # the example's own route: sort, cumulative counts by upper_bound, adjacent difference
        srt = np.sort(s)
        assert srt.tolist() == case["sorted"]
        cum = np.searchsorted(srt, np.arange(case["num_bins"]), side="right")
        assert cum.tolist() == case["cumulative"]
        assert np.diff(cum, prepend=0).tolist() == case["expected"]


def test_histogram_matches_bincount_and_invariants():
    rng = np.random.default_rng(47)
    s = rng.integers(0, 256, 100000).astype(np.uint8)
    h = oracle.histogram_even(s, 256, 0, 256)
    assert (h == np.bincount(s, minlength=256)).all() and h.sum() == s.size
    h4096 = oracle.histogram_even(s, 4096, 0, 256)  # width 1/16: only every 16th bin is hit
    assert (h4096[::16] == h).all() and h4096.sum() == s.size
    ranks = rng.zipf(1.1, 200000)
    ranks = ranks[ranks <= 4096][:100000] - 1
    f = ranks.astype(np.float32)
    assert (oracle.histogram_even(f, 4096, 0, 4096) == np.bincount(ranks, minlength=4096)).all()
    assert (oracle.histogram_even(f, 256, 0, 4096) == np.bincount(ranks // 16, minlength=256)).all()
    # out-of-range and NaN samples are dropped
    g = np.array([-1.0, 0.0, 3.999, 4.0, np.nan, 2.5], dtype=np.float32)
    assert oracle.histogram_even(g, 4, 0, 4).tolist() == [1, 0, 1, 1]
