"""Parity at the benchmark's full sizes (2^28 elements, 2^30 histogram samples), where the CPU
oracle would take minutes: every check runs on the device against an independent computation
(float64 prefix and segment sums, bincount) or a property that pins the result (sortedness,
stability, key/value association, multiset checksums)."""
import ctypes

import pytest
import torch

import thrust_amd
from thrust_amd import capi

pytestmark = pytest.mark.gpu

N = 1 << 28
FP_RTOL = 1e-5


def gen(seed):
    return torch.Generator(device="cuda").manual_seed(seed)


def run_ids(mean, seed):
    """int32 run ids with geometric run lengths of the given mean (benchmark configuration 4)."""
    if mean == 1:
        return torch.arange(N, dtype=torch.int32, device="cuda")
    heads = torch.rand(N, device="cuda", generator=gen(seed)) < (1.0 / mean)
    heads[0] = True
    return torch.cumsum(heads.to(torch.int32), 0, dtype=torch.int32) - 1


# ------------------------------------------------------------------ scan, fp32
def test_scan_f32_full_size_against_float64():
    x = torch.rand(N, dtype=torch.float32, device="cuda", generator=gen(8)) * 2 - 1
    ref = torch.cumsum(x.double(), 0)
    l1 = torch.cumsum(x.double().abs(), 0)
    got = thrust_amd.inclusive_scan(x)
    assert bool(((got.double() - ref).abs() <= FP_RTOL * l1).all())
    del got
    got = thrust_amd.exclusive_scan(x, init=0.5)
    # exclusive[i] = 0.5 + inclusive[i-1]
    assert float(got[0].item()) == 0.5
    assert bool(((got[1:].double() - (ref[:-1] + 0.5)).abs() <= FP_RTOL * (l1[:-1] + 0.5)).all())


# ------------------------------------------------------------------ reduce_by_key
@pytest.mark.parametrize("mean", [1, 8, 512])
def test_reduce_by_key_f32_full_size_against_float64_segment_sums(mean):
    keys = run_ids(mean, 20 + mean)
    vals = torch.randn(N, dtype=torch.float32, device="cuda", generator=gen(31))
    r = int(keys[-1].item()) + 1
    gk, gv = thrust_amd.reduce_by_key(keys, vals)
    assert gk.numel() == r
    assert torch.equal(gk, torch.arange(r, dtype=torch.int32, device="cuda"))
    idx = keys.long()
    ref = torch.zeros(r, dtype=torch.float64, device="cuda").index_add_(0, idx, vals.double())
    l1 = torch.zeros(r, dtype=torch.float64, device="cuda").index_add_(0, idx, vals.double().abs())
    assert bool(((gv.double() - ref).abs() <= FP_RTOL * l1 + 1e-30).all())


@pytest.mark.parametrize("mean", [1, 8, 512])
def test_reduce_by_key_i32_full_size_exact(mean):
    keys = run_ids(mean, 20 + mean)
    vals = torch.randint(-1000, 1001, (N,), dtype=torch.int32, device="cuda", generator=gen(9))
    r = int(keys[-1].item()) + 1
    gk, gv = thrust_amd.reduce_by_key(keys, vals)
    assert gk.numel() == r
    assert torch.equal(gk, torch.arange(r, dtype=torch.int32, device="cuda"))
    ref = torch.zeros(r, dtype=torch.int64, device="cuda").index_add_(0, keys.long(), vals.long())
    assert torch.equal(gv.long(), ref)  # |sum| of a run stays far below 2^31 here


def test_scan_by_key_i32_full_size_exact():
    keys = run_ids(8, 28)
    vals = torch.randint(-1000, 1001, (N,), dtype=torch.int32, device="cuda", generator=gen(9))
    got = thrust_amd.inclusive_scan_by_key(keys, vals).long()
    # segmented inclusive scan = global prefix sum minus the prefix sum just before the run's head
    c = torch.cumsum(vals.long(), 0)
    head = torch.ones(N, dtype=torch.bool, device="cuda")
    head[1:] = keys[1:] != keys[:-1]
    before_head = (c - vals.long())[head]  # one entry per run
    assert torch.equal(got, c - before_head[keys.long()])


def test_by_key_beyond_2p31_elements():
    # more elements than a signed 32-bit offset holds (the reference dispatches to 64-bit offsets
    # there, thrust/system/cuda/detail/dispatch.h:29-78); runs of 512 ones have closed forms
    n = (1 << 31) + 777
    keys = (torch.arange(n, dtype=torch.int64, device="cuda") >> 9).to(torch.int32)
    vals = torch.ones(n, dtype=torch.int32, device="cuda")
    gk, gv = thrust_amd.reduce_by_key(keys, vals)
    r = (n + 511) // 512
    assert gk.numel() == r
    assert torch.equal(gk, torch.arange(r, dtype=torch.int32, device="cuda"))
    assert bool((gv[:-1] == 512).all()) and int(gv[-1].item()) == n - 512 * (r - 1)
    del gk, gv
    out = thrust_amd.inclusive_scan_by_key(keys, vals)
    assert int(out[-1].item()) == n - 512 * (r - 1) and int(out[(1 << 31) - 1].item()) == 512
    pos = torch.arange(n - (1 << 20), n, dtype=torch.int64, device="cuda")
    assert torch.equal(out[-(1 << 20):].long(), (pos & 511) + 1)
    assert torch.equal(out[:1 << 20].long(), (torch.arange(1 << 20, dtype=torch.int64, device="cuda") & 511) + 1)


# ------------------------------------------------------------------ sort_by_key u64 + u32
def unsigned_order(k):
    """int64 whose signed order is the unsigned order of the 64-bit patterns in k."""
    return k ^ torch.tensor(-2**63, dtype=torch.int64, device=k.device)


@pytest.mark.parametrize("words", [0, 1, 2, 3, 4])
def test_sort_by_key_u64_u32_full_size_sorted_stable_and_associated(words):
    # keys = AND of `words` uniform 64-bit words (fewer effective bits as words grows); 0 = all equal
    if words == 0:
        k0 = torch.full((N,), 42, dtype=torch.int64, device="cuda")
    else:
        k0 = torch.randint(-2**63, 2**63 - 1, (N,), dtype=torch.int64, device="cuda", generator=gen(1338))
        for w in range(1, words):
            k0 &= torch.randint(-2**63, 2**63 - 1, (N,), dtype=torch.int64, device="cuda", generator=gen(1338 + w))
    k = k0.clone()
    v = torch.arange(N, dtype=torch.int32, device="cuda")
    thrust_amd.sort_by_key(k.view(torch.uint64), v)
    assert torch.equal(k0[v.long()], k)  # every value still names its key: v is a permutation consistent with k
    u = unsigned_order(k)
    assert bool((u[1:] >= u[:-1]).all())  # ascending as unsigned 64-bit
    assert bool(((u[1:] > u[:-1]) | (v[1:] > v[:-1])).all())  # equal keys keep their input order (so v is a permutation)
    c = ctypes.c_ulonglong(1)
    assert capi.lib().thrust_cdna4_lookback_timeouts(ctypes.byref(c)) == 0 and c.value == 0


def test_sort_f32_keys_full_size_total_order():
    k0 = torch.randn(N, dtype=torch.float32, device="cuda", generator=gen(77))
    tiny = float(torch.finfo(torch.float32).tiny)
    specials = torch.tensor([0.0, -0.0, tiny / 4, -tiny / 4, tiny / 1024, float("inf"), float("-inf")],
                            dtype=torch.float32, device="cuda")
    pos = torch.randint(0, N, (7000,), device="cuda", generator=gen(78))
    k0[pos] = specials.repeat(1000)
    k = k0.clone()
    thrust_amd.sort(k)
    bits = k.view(torch.int32)
    # signed integer whose order is the reference's float order (-0 before +0, denormals in place):
    # negatives have their low 31 bits flipped (sequential/stable_radix_sort.inl:120-126)
    s = bits ^ ((bits >> 31) & 0x7FFFFFFF)
    assert bool((s[1:] >= s[:-1]).all())
    b0 = k0.view(torch.int32)
    assert int(bits.sum(dtype=torch.int64).item()) == int(b0.sum(dtype=torch.int64).item())
    s0 = b0 ^ ((b0 >> 31) & 0x7FFFFFFF)
    assert int(s.min().item()) == int(s0.min().item()) and int(s.max().item()) == int(s0.max().item())
    # the multiset is preserved: both sides histogram identically under a hash of the bit pattern
    h = lambda t: torch.bincount(((t.long() * 2654435761) >> 7) & 0xFFFF, minlength=65536)
    assert torch.equal(h(bits), h(b0))


# ------------------------------------------------------------------ histogram, 2^30 samples
@pytest.mark.parametrize("bins", [256, 4096])
def test_histogram_f32_zipf_full_size_against_bincount(bins):
    m = 1 << 30
    w = 1.0 / torch.arange(1, 4097, dtype=torch.float64, device="cuda") ** 1.1
    cdf = torch.cumsum(w / w.sum(), 0).to(torch.float32)
    f = torch.empty(m, dtype=torch.float32, device="cuda")
    ref = torch.zeros(bins, dtype=torch.int64, device="cuda")
    chunk = 1 << 26
    for i in range(m // chunk):  # in pieces: searchsorted returns int64
        u = torch.rand(chunk, dtype=torch.float32, device="cuda", generator=gen(12 + i))
        rank = torch.searchsorted(cdf, u).clamp_(max=4095)
        f[i * chunk:(i + 1) * chunk] = rank.to(torch.float32)
        ref += torch.bincount(rank // (4096 // bins), minlength=bins)
    got = thrust_amd.histogram_even(f, bins, 0.0, 4096.0)
    assert torch.equal(got.long(), ref)


@pytest.mark.parametrize("bins", [256, 4096])
def test_histogram_u8_full_size_against_bincount(bins):
    m = 1 << 30
    s = torch.randint(0, 256, (m,), dtype=torch.uint8, device="cuda", generator=gen(11))
    got = thrust_amd.histogram_even(s, bins, 0.0, 256.0)
    ref = torch.zeros(bins, dtype=torch.int64, device="cuda")
    per = torch.zeros(256, dtype=torch.int64, device="cuda")
    for piece in s.view(16, -1):
        per += torch.bincount(piece.long(), minlength=256)
    ref[torch.arange(256, device="cuda") * (bins // 256)] = per  # value b falls in bin b * bins / 256
    assert torch.equal(got.long(), ref)
