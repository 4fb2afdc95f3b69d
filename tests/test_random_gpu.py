"""Randomised cross-check of the C-ABI algorithms against the oracle: sizes, element types,
operators, run lengths, misaligned views and the look-back patience are all drawn from a seeded
generator, so every run checks the same few hundred cases (bit-exact; integer values only, the
floating-point tolerances have their own tests)."""
import numpy as np
import pytest
import torch

import oracle
import thrust_amd
from conftest import INT_DTYPES, random_ints, same_bits
from gpu_util import dev, host
from thrust_amd import capi

pytestmark = pytest.mark.gpu

OPS = ["plus", "maximum", "minimum", "multiplies"]


def draw_size(rng):
    kind = rng.integers(0, 4)
    if kind == 0:
        return int(rng.integers(0, 300))
    if kind == 1:  # around tile boundaries of the scan (32768), by-key (16384 / 8192) and sort tiles
        return int(rng.choice([8192, 16384, 32768, 65536, 131072]) * rng.integers(1, 5) + rng.integers(-3, 4))
    if kind == 2:
        return int(rng.integers(300, 200_000))
    return int(rng.integers(200_000, 3_000_000))


def misaligned(arr, shift):
    """A device copy of arr that starts `shift` elements into a larger allocation."""
    padded = np.concatenate([np.zeros(shift, dtype=arr.dtype), arr])
    return dev(padded)[shift:]


def runs_of(rng, n, kd):
    if n == 0:
        return np.zeros(0, dtype=kd)
    mean = float(rng.choice([1, 2, 8, 100, 5000]))
    heads = rng.random(n) < 1.0 / mean
    ids = np.cumsum(heads)
    return (ids % 119).astype(kd) if np.dtype(kd).itemsize == 1 else ids.astype(kd)


@pytest.mark.parametrize("seed", range(6))
def test_random_scans(seed):
    rng = np.random.default_rng(1000 + seed)
    L = capi.lib()
    for case in range(20):
        n = draw_size(rng)
        dt = INT_DTYPES[rng.integers(0, len(INT_DTYPES))]
        op = OPS[rng.integers(0, 4)]
        exclusive = bool(rng.integers(0, 2))
        shift = int(rng.integers(0, 4))
        in_place = bool(rng.integers(0, 3) == 0)
        previous = L.thrust_cdna4_set_lookback_patience(int(rng.choice([0, 1, 256])))
        try:
            x = random_ints(seed * 100 + case, n, dt)
            if op == "multiplies":
                x = (x % 3 + 1).astype(dt)  # products wrap anyway; keep them non-zero
            d = misaligned(x, shift)
            init = 3 if exclusive else None
            if exclusive:
                got = thrust_amd.exclusive_scan(d, out=d if in_place else None, init=init, op=op)
            else:
                got = thrust_amd.inclusive_scan(d, out=d if in_place else None, op=op)
            ref = oracle.scan(x, op, exclusive=exclusive, init=init)
            assert same_bits(host(got), ref), (seed, case, n, dt, op, exclusive, shift, in_place)
        finally:
            L.thrust_cdna4_set_lookback_patience(previous)


@pytest.mark.parametrize("seed", range(6))
def test_random_by_key(seed):
    rng = np.random.default_rng(2000 + seed)
    L = capi.lib()
    for case in range(14):
        n = draw_size(rng)
        kd = INT_DTYPES[rng.integers(0, len(INT_DTYPES))]
        vd = INT_DTYPES[rng.integers(0, len(INT_DTYPES))]
        op = OPS[rng.integers(0, 3)]
        shift = int(rng.integers(0, 4))
        previous = L.thrust_cdna4_set_lookback_patience(int(rng.choice([0, 1, 256])))
        try:
            k = runs_of(rng, n, kd)
            v = random_ints(seed * 100 + case + 7, n, vd)
            dk, dv = misaligned(k, shift), misaligned(v, int(rng.integers(0, 4)))
            exclusive = bool(rng.integers(0, 2))
            if exclusive:
                got = thrust_amd.exclusive_scan_by_key(dk, dv, init=5, op=op)
            else:
                got = thrust_amd.inclusive_scan_by_key(dk, dv, op=op)
            assert same_bits(host(got), oracle.scan_by_key(k, v, op, exclusive=exclusive, init=5 if exclusive else None)), \
                (seed, case, n, kd, vd, op, exclusive)
            gk, gv = thrust_amd.reduce_by_key(dk, dv, op=op)
            rk, rv = oracle.reduce_by_key(k, v, op)
            assert same_bits(host(gk), rk) and same_bits(host(gv), rv), (seed, case, n, kd, vd, op)
        finally:
            L.thrust_cdna4_set_lookback_patience(previous)


@pytest.mark.parametrize("seed", range(4))
def test_random_sorts(seed):
    rng = np.random.default_rng(3000 + seed)
    for case in range(12):
        n = draw_size(rng)
        kd = INT_DTYPES[rng.integers(0, len(INT_DTYPES))]
        descending = bool(rng.integers(0, 2))
        bits = int(rng.integers(1, 8 * np.dtype(kd).itemsize + 1))
        k = random_ints(seed * 100 + case + 3, n, kd)
        if bits < 8 * np.dtype(kd).itemsize:
            k = (k.astype(np.uint64) & np.uint64((1 << bits) - 1)).astype(kd)
        if rng.integers(0, 2):
            d = misaligned(k, int(rng.integers(0, 4)))
            thrust_amd.sort(d, descending)
            assert same_bits(host(d), oracle.sort_keys(k, descending)), (seed, case, n, kd, descending, bits)
        else:
            vd = [np.uint8, np.uint16, np.uint32, np.uint64][rng.integers(0, 4)]
            v = random_ints(seed + case, n, vd)
            dk, dv = misaligned(k, int(rng.integers(0, 4))), misaligned(v, int(rng.integers(0, 4)))
            thrust_amd.sort_by_key(dk, dv, descending)
            rk, rv = oracle.sort_pairs(k, v, descending)
            assert same_bits(host(dk), rk) and same_bits(host(dv), rv), (seed, case, n, kd, vd, descending, bits)
