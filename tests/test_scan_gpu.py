"""GPU parity of thrust_cdna4_scan against the oracle: integers bit-exact, floating point
within 1e-5 of the running L1 norm (a reassociated sum cannot match the serial fold bit for
bit; the bound is relative to sum |x_j| because prefix sums cross zero)."""
import numpy as np
import pytest
import torch

import oracle
import thrust_amd
from conftest import INT_DTYPES, SIZES, random_ints, same_bits
import gpu_util
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

FP_RTOL = 1e-5


def test_scan_kat(kat):
    for case in kat["scan"]:
        for dt in [np.int8, np.int16, np.int32, np.int64, np.float32, np.float64]:
            x = dev(np.array(case["input"], dtype=dt))
            if case["exclusive"]:
                out = thrust_amd.exclusive_scan(x, init=case["init"], op=case["op"])
            else:
                out = thrust_amd.inclusive_scan(x, op=case["op"])
            assert host(out).tolist() == case["expected"], (case["source"], dt)
            assert host(x).tolist() == case["input"]  # input untouched
            if case["exclusive"]:
                thrust_amd.exclusive_scan(x, out=x, init=case["init"], op=case["op"])  # in place
            else:
                thrust_amd.inclusive_scan(x, out=x, op=case["op"])
            assert host(x).tolist() == case["expected"], (case["source"], dt, "in place")


def test_scan_i32_size_ladder():
    for n in SIZES:
        x = (random_ints(n, n, np.uint32) % 16).astype(np.int32)
        d = dev(x)
        assert same_bits(host(thrust_amd.inclusive_scan(d)), oracle.scan(x)), n
        assert same_bits(host(thrust_amd.exclusive_scan(d, init=3)), oracle.scan(x, exclusive=True, init=3)), n


@pytest.mark.parametrize("dtype", INT_DTYPES)
@pytest.mark.parametrize("op", ["plus", "multiplies", "maximum", "minimum"])
def test_scan_int_types_and_ops(dtype, op):
    for n in [1, 65, 4097, 100003]:
        x = random_ints(5 + n, n, dtype)
        d = dev(x)
        assert same_bits(host(thrust_amd.inclusive_scan(d, op=op)), oracle.scan(x, op)), n
        assert same_bits(host(thrust_amd.exclusive_scan(d, init=7, op=op)),
                         oracle.scan(x, op, exclusive=True, init=7)), n


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_scan_float_plus_tolerance(dtype):
    for n in [1, 100, 4097, 1 << 20]:
        x = np.random.default_rng(n).uniform(-1, 1, n).astype(dtype)
        d = dev(x)
        ref = np.cumsum(x.astype(np.float64))
        l1 = np.cumsum(np.abs(x.astype(np.float64)))
        got = host(thrust_amd.inclusive_scan(d)).astype(np.float64)
        assert (np.abs(got - ref) <= FP_RTOL * l1).all(), n
        serial = oracle.scan(x).astype(np.float64)  # the reference's own left fold
        assert (np.abs(got - serial) <= FP_RTOL * l1).all(), n
        got = host(thrust_amd.exclusive_scan(d, init=0.5)).astype(np.float64)
        ref_e = np.concatenate([[0.0], ref[:-1]]) + 0.5
        assert (np.abs(got - ref_e) <= FP_RTOL * (l1 + 0.5)).all(), n


def test_scan_float_max_min_exact():
    x = np.random.default_rng(2).standard_normal(200001).astype(np.float32)
    d = dev(x)
    assert same_bits(host(thrust_amd.inclusive_scan(d, op="maximum")), np.maximum.accumulate(x))
    assert same_bits(host(thrust_amd.inclusive_scan(d, op="minimum")), np.minimum.accumulate(x))


def test_scan_unaligned_in_place():
    x = (random_ints(9, 70001, np.uint32) % 16).astype(np.int32)
    d = dev(x)
    v = d[1:]
    thrust_amd.inclusive_scan(v, out=v)
    assert same_bits(host(v), oracle.scan(x[1:]))
    assert host(d)[0] == x[0]


@pytest.mark.needs_device
def test_scan_full_size_closed_forms():
    # 2^28 elements (benchmark configuration 2): constants have closed-form scans
    n = 1 << 28
    ones = torch.ones(n, dtype=torch.int32, device=gpu_util.DEVICE)
    out = thrust_amd.inclusive_scan(ones)
    assert torch.equal(out, torch.arange(1, n + 1, dtype=torch.int32, device=gpu_util.DEVICE))
    thrust_amd.exclusive_scan(ones, out=ones, init=0)  # in place
    assert torch.equal(ones, torch.arange(0, n, dtype=torch.int32, device=gpu_util.DEVICE))
    del ones, out
    g = torch.Generator(device=gpu_util.DEVICE).manual_seed(5)
    x = torch.randint(0, 16, (n,), dtype=torch.int32, device=gpu_util.DEVICE, generator=g)
    incl = thrust_amd.inclusive_scan(x)
    excl = thrust_amd.exclusive_scan(x, init=0)
    assert torch.equal(incl - excl, x)  # inclusive[i] - exclusive[i] == x[i]
    assert int(incl[-1].item()) == int(x.sum(dtype=torch.int64).item())
    assert bool((incl[1:] >= incl[:-1]).all())


def test_scan_repeat_determinism_ints():
    x = dev((random_ints(4, 1 << 22, np.uint32) % 16).astype(np.int32))
    first = host(thrust_amd.inclusive_scan(x)).tobytes()
    for _ in range(5):
        assert host(thrust_amd.inclusive_scan(x)).tobytes() == first


@pytest.fixture
def no_patience():
    """Look-back never waits: every tile descriptor that is not there yet is recomputed from the
    input by the workgroup that needs it (the forward-progress path of the ticketless kernels)."""
    from thrust_amd import capi
    L = capi.lib()
    previous = L.thrust_cdna4_set_lookback_patience(0)
    yield
    L.thrust_cdna4_set_lookback_patience(previous)


@pytest.fixture
def tile0_publishes_late():
    """Tile 0 sleeps ~10 ms (a bounded number of sleeps) before it publishes its descriptor, so
    with patience 0 every later tile finds it missing at the first AND at the second look and
    has to use the aggregate it recomputed from the input.  Every kernel still exits normally."""
    from thrust_amd import capi
    L = capi.lib()
    previous = L.thrust_cdna4_set_test_publish_delay(3000)
    yield
    L.thrust_cdna4_set_test_publish_delay(previous)


@pytest.mark.parametrize("op", ["plus", "multiplies", "maximum", "minimum"])
def test_exclusive_scan_init_survives_a_recomputed_tile0(no_patience, tile0_publishes_late, op):
    # semantics: thrust/system/detail/sequential/scan.h:95-111 (out[0] = init, then init op x0 ...)
    for dtype, n in [(np.int32, 200_003), (np.int64, 70_001), (np.uint8, 300_000), (np.int16, 300_001)]:
        x = random_ints(77 + n, n, dtype)
        d = dev(x)
        for init in (7, 0):
            got = host(thrust_amd.exclusive_scan(d, init=init, op=op))
            assert same_bits(got, oracle.scan(x, op, exclusive=True, init=init)), (dtype, n, init)
        assert same_bits(host(thrust_amd.inclusive_scan(d, op=op)), oracle.scan(x, op)), (dtype, n)
    f = np.random.default_rng(8).uniform(-1, 1, 150_001).astype(np.float32)
    got = host(thrust_amd.exclusive_scan(dev(f), init=0.5, op="plus")).astype(np.float64)
    ref = np.concatenate([[0.0], np.cumsum(f.astype(np.float64))[:-1]]) + 0.5
    l1 = np.concatenate([[0.0], np.cumsum(np.abs(f.astype(np.float64)))[:-1]]) + 0.5
    assert (np.abs(got - ref) <= FP_RTOL * l1).all()


def test_scan_recompute_path_matches_oracle(no_patience):
    for n in [1, 4097, 32768, 32769, 200_003, (1 << 22) + 5]:
        x = random_ints(50 + n, n, np.int32)
        d = dev(x)
        assert same_bits(host(thrust_amd.inclusive_scan(d)), oracle.scan(x, "plus")), n
        assert same_bits(host(thrust_amd.exclusive_scan(d, init=7)), oracle.scan(x, "plus", exclusive=True, init=7)), n
    x = random_ints(9, 1 << 21, np.uint64)
    assert same_bits(host(thrust_amd.inclusive_scan(dev(x), op="maximum")), oracle.scan(x, "maximum"))
    f = np.random.default_rng(3).uniform(-1, 1, 300_001).astype(np.float32)
    got = host(thrust_amd.inclusive_scan(dev(f))).astype(np.float64)
    ref = np.cumsum(f.astype(np.float64))
    assert (np.abs(got - ref) <= FP_RTOL * np.cumsum(np.abs(f.astype(np.float64)))).all()


@pytest.mark.needs_device
def test_scan_full_size_recompute_path(no_patience):
    n = 1 << 28
    x = torch.ones(n, dtype=torch.int32, device=gpu_util.DEVICE)
    out = thrust_amd.inclusive_scan(x)
    assert int(out[-1].item()) == n and int(out[12345678].item()) == 12345679
    assert bool((out[1:] - out[:-1] == 1).all())


def test_scan_in_place_takes_the_ticket_path_and_out_of_place_does_not():
    # both paths give the same bits; partially overlapping ranges count as in place
    x = random_ints(123, (1 << 20) + 3, np.int32)
    ref = oracle.scan(x, "plus")
    d = dev(x)
    assert same_bits(host(thrust_amd.inclusive_scan(d)), ref)
    thrust_amd.inclusive_scan(d, out=d)
    assert same_bits(host(d), ref)
    buf = torch.empty(x.size + 64, dtype=torch.int32, device=gpu_util.DEVICE)
    src = buf[64:]
    src.copy_(dev(x))
    dst = buf[:x.size]  # starts 256 bytes before the input
    thrust_amd.inclusive_scan(src, out=dst)
    assert same_bits(host(dst), ref)


def _with_nans(rng, n, where, dt):
    x = rng.uniform(-5, 5, n).astype(dt)
    x[rng.random(n) < 0.05] = dt(-np.inf)
    x[rng.random(n) < 0.05] = dt(np.inf)
    x[rng.random(n) < 0.04] = dt(0.0)   # ties between +0 and -0 show which operand a fold keeps
    x[rng.random(n) < 0.04] = dt(-0.0)
    if where == "first":
        x[0] = np.nan
    elif where == "middle" and n > 2:
        x[n // 2] = np.nan
        x[1] = np.nan
    elif where == "many":
        x[rng.random(n) < 0.3] = np.nan
        x[0] = dt(1.0)
    elif where == "many_and_first":
        x[rng.random(n) < 0.3] = np.nan
        x[0] = np.nan
    elif where == "all":
        x[:] = np.nan
    # NaNs of both signs and with different payloads: the fold must hand on the very NaN it met
    nan = np.isnan(x)
    u = x.view(np.uint32 if dt == np.float32 else np.uint64)
    width = u.dtype.itemsize * 8
    u[nan] ^= (rng.integers(0, 1 << 20, int(nan.sum())).astype(u.dtype)
               | (rng.integers(0, 2, int(nan.sum())).astype(u.dtype) << u.dtype.type(width - 1)))
    return x


@pytest.mark.parametrize("op", ["maximum", "minimum"])
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_float_extrema_scans_with_nans_are_the_serial_fold(dt, op):
    """thrust::maximum is a < b ? b : a: the serial fold (thrust/system/detail/sequential/scan.h:54-72)
    keeps a NaN that starts it and skips NaNs met later.  thrust::minimum is a < b ? a : b: the fold
    restarts at every NaN (the NaN replaces the accumulator, the next element replaces the NaN).  The
    kernel must give the same bits whatever its grouping: NaN first, in the middle, scattered,
    everywhere; a NaN `init`; several tiles; in place."""
    rng = np.random.default_rng(11)
    for n in (1, 2, 5, 4097, 70001, 300007):
        for where in ("none", "first", "middle", "many", "many_and_first", "all"):
            x = _with_nans(rng, n, where, dt)
            d = dev(x)
            assert same_bits(host(thrust_amd.inclusive_scan(d, op=op)), oracle.scan(x, op=op)), (n, where)
            for init in (dt(0.5), dt(np.nan), dt(-np.inf)):
                assert same_bits(host(thrust_amd.exclusive_scan(d, init=init, op=op)),
                                 oracle.scan(x, op=op, exclusive=True, init=init)), (n, where, init)
            y = dev(x)
            thrust_amd.inclusive_scan(y, out=y, op=op)  # in place: tiles by ticket
            assert same_bits(host(y), oracle.scan(x, op=op)), (n, where, "in place")
            y = dev(x)
            thrust_amd.exclusive_scan(y, out=y, init=dt(np.nan), op=op)
            assert same_bits(host(y), oracle.scan(x, op=op, exclusive=True, init=dt(np.nan))), (n, where, "in place, NaN init")


def test_float_maximum_scan_with_nans_on_the_recompute_path(no_patience, tile0_publishes_late):
    rng = np.random.default_rng(12)
    n = 32768 * 3 + 77
    for where in ("first", "many", "many_and_first"):
        x = _with_nans(rng, n, where, np.float32)
        d = dev(x)
        assert same_bits(host(thrust_amd.inclusive_scan(d, op="maximum")), oracle.scan(x, op="maximum")), where
        assert same_bits(host(thrust_amd.exclusive_scan(d, init=np.float32(2.0), op="maximum")),
                         oracle.scan(x, op="maximum", exclusive=True, init=np.float32(2.0))), where


def _zeros_of_both_signs(rng, n, dt, op):
    """Mostly +0 and -0, the rest on the side that never wins: every result is a zero whose SIGN tells
    which operand the fold kept (maximum keeps the first of equals, minimum the last)."""
    x = np.where(rng.random(n) < 0.5, dt(0.0), dt(-0.0)).astype(dt)
    losers = rng.random(n) < 0.3
    x[losers] = (-1 if op == "maximum" else 1) * rng.uniform(1, 5, int(losers.sum())).astype(dt)
    return x


@pytest.mark.parametrize("op", ["maximum", "minimum"])
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_float_extrema_scans_keep_the_zero_the_serial_fold_keeps(dt, op):
    rng = np.random.default_rng(31)
    for n in (7, 4097, 70001, 300007):
        x = _zeros_of_both_signs(rng, n, dt, op)
        d = dev(x)
        assert same_bits(host(thrust_amd.inclusive_scan(d, op=op)), oracle.scan(x, op=op)), n
        for init in (dt(0.0), dt(-0.0)):
            assert same_bits(host(thrust_amd.exclusive_scan(d, init=init, op=op)),
                             oracle.scan(x, op=op, exclusive=True, init=init)), (n, init)
        y = dev(x)
        thrust_amd.exclusive_scan(y, out=y, init=dt(-0.0), op=op)  # in place: tiles by ticket
        assert same_bits(host(y), oracle.scan(x, op=op, exclusive=True, init=dt(-0.0))), (n, "in place")


@pytest.mark.parametrize("op", ["maximum", "minimum"])
def test_float_extrema_scans_keep_that_zero_on_the_recompute_path(no_patience, tile0_publishes_late, op):
    rng = np.random.default_rng(32)
    n = 32768 * 4 + 77
    for dt in (np.float32, np.float64):
        x = _zeros_of_both_signs(rng, n, dt, op)
        d = dev(x)
        assert same_bits(host(thrust_amd.inclusive_scan(d, op=op)), oracle.scan(x, op=op)), dt
        assert same_bits(host(thrust_amd.exclusive_scan(d, init=dt(-0.0), op=op)),
                         oracle.scan(x, op=op, exclusive=True, init=dt(-0.0))), dt
