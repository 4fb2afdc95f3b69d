"""GPU parity of thrust_cdna4_histogram_even against the oracle's counting loop (bit-exact)."""
import numpy as np
import pytest
import torch

import oracle
import thrust_amd
from conftest import ALL_DTYPES, same_bits
import gpu_util
from gpu_util import dev, host

pytestmark = pytest.mark.gpu


def counts(t):
    return host(t).view(np.uint32)


def test_histogram_kat(kat):
    case = kat["histogram"][0]
    for dt in ALL_DTYPES:
        s = dev(np.array(case["samples"], dtype=dt))
        got = thrust_amd.histogram_even(s, case["num_bins"], case["lower"], case["upper"])
        assert counts(got).tolist() == case["expected"], dt


@pytest.mark.parametrize("bins", [256, 4096])
def test_histogram_u8_uniform(bins):
    for n in [0, 1, 1000, (1 << 22) + 5]:
        s = np.random.default_rng(n).integers(0, 256, n).astype(np.uint8)
        got = counts(thrust_amd.histogram_even(dev(s), bins, 0, 256))
        assert same_bits(got, oracle.histogram_even(s, bins, 0, 256)), n
        assert got.sum() == n


@pytest.mark.parametrize("bins", [256, 4096])
def test_histogram_f32_zipf(bins):
    rng = np.random.default_rng(1)
    r = rng.zipf(1.1, 6_000_000)
    r = (r[r <= 4096] - 1)[: (1 << 21) + 3]
    s = r.astype(np.float32)
    got = counts(thrust_amd.histogram_even(dev(s), bins, 0, 4096))
    assert same_bits(got, oracle.histogram_even(s, bins, 0, 4096))
    assert same_bits(got, np.bincount(r // (4096 // bins), minlength=bins).astype(np.uint32))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_histogram_all_types_general_ranges(dtype):
    rng = np.random.default_rng(5)
    n = 100003
    if np.dtype(dtype).kind == "f":
        s = (rng.standard_normal(n) * 50).astype(dtype)
        s[:4] = [np.nan, np.inf, -np.inf, 0.0]
    else:
        info = np.iinfo(dtype)
        s = rng.integers(max(info.min, -300), min(info.max, 300), n, endpoint=True).astype(dtype)
    for bins, lo, hi in [(7, -100.0, 100.0), (256, -128.0, 128.0), (257, -100.0, 157.0), (512, -256.0, 256.0),
                         (513, -256.0, 257.0), (1000, 0.0, 250.0), (8192, -300.0, 300.0), (2048, -64.0, 64.0), (2049, -64.0, 64.0),
                         (4097, -300.0, 300.0), (8193, -300.0, 300.0), (16384, -300.0, 300.0), (70000, -300.5, 300.5)]:
        got = counts(thrust_amd.histogram_even(dev(s), bins, lo, hi))
        assert same_bits(got, oracle.histogram_even(s, bins, lo, hi)), (bins, lo, hi)


@pytest.mark.needs_device
def test_histogram_full_size_closed_form():
    # 2^30 u8 samples i % 256: every bin holds exactly 2^22
    n = 1 << 30
    s = (torch.arange(n, dtype=torch.int32, device=gpu_util.DEVICE) & 255).to(torch.uint8)
    got = counts(thrust_amd.histogram_even(s, 256, 0, 256))
    assert (got == (1 << 22)).all()
