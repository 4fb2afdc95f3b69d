#!/usr/bin/env python3
"""Benchmark of the gfx950 Thrust device system on one MI355X.

A "step" is one thrust::sort of 2^28 uniformly random uint32 keys (seed 1337) through the
C ABI, input already resident in HBM; the unsorted input is restored between steps outside
the timed region.  Prints ONE JSON line.  The other workloads of the headline metric
(u64+u32 sort_by_key, scan, reduce_by_key, histogram) are measured the same way with a few
repetitions each and reported under "extras".

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# measured HBM traffic of one onesweep launch over 2^28 uint32 keys
# (profiles/onesweep_u32_sort_2p28_and_extras.md)
ONESWEEP_U32_TRAFFIC_BYTES = 2.213e9


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--log2n", type=int, default=28, help="log2 of the element count (default 28)")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only", default="", help="run a single extra workload by name (profiling aid)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)",
              file=sys.stderr)
        sys.exit(2)

    import ctypes

    import numpy as np
    import torch

    import thrust_amd
    from thrust_amd import capi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    L = capi.lib()
    dev = torch.device("cuda:0")
    n = 1 << args.log2n
    stream = torch.cuda.current_stream()
    sp = ctypes.c_void_p(stream.cuda_stream)

    def gen(seed):
        return torch.Generator(device=dev).manual_seed(seed)

    def timed(fn, restore, steps, warmup):
        """Runs restore(); fn() `warmup`+`steps` times; returns per-step ms from HIP events
        recorded on the launch stream around fn() only."""
        for _ in range(warmup):
            restore()
            fn()
        torch.cuda.synchronize()
        evs = []
        for _ in range(steps):
            restore()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            fn()
            e1.record(stream)
            evs.append((e0, e1))
        torch.cuda.synchronize()
        return [a.elapsed_time(b) for a, b in evs]

    def kernel_ms(fn, restore, kernel, reps=3):
        """Average launch duration of `kernel` from the library's launch log (HIP events on
        the launch stream around each launch)."""
        L.thrust_cdna4_profile_enable(1)
        for _ in range(reps):
            restore()
            fn()
        torch.cuda.synchronize()
        recs = [ms for name, ms in capi.profile_records() if name == kernel]
        L.thrust_cdna4_profile_enable(0)
        return sum(recs) / len(recs), len(recs)

    # ------------------------------------------------------------------ headline: sort u32
    def two_phase(call):
        nb = ctypes.c_size_t(0)
        capi.check(call(None, nb), "size query")
        tmp = torch.empty(max(nb.value, 1), dtype=torch.uint8, device=dev)
        return tmp, nb

    results = {}

    def run_sort_u32(steps, warmup):
        src = torch.randint(-2**31, 2**31, (n,), dtype=torch.int32, device=dev, generator=gen(1337))
        keys = torch.empty_like(src)
        kp = ctypes.c_void_p(keys.data_ptr())
        call = lambda t, nb: L.thrust_cdna4_sort_keys(t, ctypes.byref(nb), capi.U32, kp, n, 0, sp)
        tmp, nb = two_phase(call)
        tp = ctypes.c_void_p(tmp.data_ptr())
        fn = lambda: capi.check(call(tp, nb), "sort_keys")
        restore = lambda: keys.copy_(src)
        ms = timed(fn, restore, steps, warmup)
        kms, launches = kernel_ms(fn, restore, "onesweep_kernel")
        # parity property at full size: sorted, multiset preserved
        restore(); fn(); torch.cuda.synchronize()
        hk = keys.cpu().numpy().view(np.uint32)
        assert (hk[1:] >= hk[:-1]).all(), "sort output not sorted"
        assert int(hk.view(np.int32).sum(dtype=np.int64)) == int(src.sum(dtype=torch.int64).item())
        return ms, kms, launches

    t_wall0 = time.time()
    ms_list, onesweep_ms, onesweep_launches = run_sort_u32(args.steps, args.warmup)
    ms_per_step = sum(ms_list) / len(ms_list)
    gkeys = n / ms_per_step / 1e6
    sort_bytes = 36.0 * n  # 4 * (1 + 2*4) per key
    # dominant kernel: one onesweep pass reads and writes every key once
    onesweep_bytes = 8.0 * n
    onesweep_gbs = onesweep_bytes / onesweep_ms / 1e6

    # ------------------------------------------------------------------ extras
    extras = {}

    def add_extra(name, unit_items, ms, alg_bytes, unit):
        med = float(np.median(ms))
        extras[name] = {
            "value": round(unit_items / med / 1e6, 3), "unit": unit, "ms": round(med, 4),
            "algorithmic_bytes": alg_bytes,
            "roofline_frac": round(alg_bytes / med / 1e6 / HBM_PEAK_GBS, 4),
        }

    def extra_sort_pairs():
        k0 = torch.randint(-2**63, 2**63 - 1, (n,), dtype=torch.int64, device=dev, generator=gen(1338))
        v0 = torch.arange(n, dtype=torch.int32, device=dev)
        k = torch.empty_like(k0)
        v = torch.empty_like(v0)
        call = lambda t, nb: L.thrust_cdna4_sort_pairs(t, ctypes.byref(nb), capi.U64,
                                                        ctypes.c_void_p(k.data_ptr()), 4,
                                                        ctypes.c_void_p(v.data_ptr()), n, 0, sp)
        tmp, nb = two_phase(call)
        tp = ctypes.c_void_p(tmp.data_ptr())
        fn = lambda: capi.check(call(tp, nb), "sort_pairs")

        def restore():
            k.copy_(k0)
            v.copy_(v0)
        ms = timed(fn, restore, 5, 1)
        assert torch.equal(k0[v.long()], k), "sort_by_key: values are not the permutation of the keys"
        add_extra("sort_by_key_u64_u32", n, ms, 200.0 * n, "Gkeys/s")
        # the same call on keys whose upper bytes are all alike (64-bit keys that hold 32-bit numbers;
        # all keys equal): places where every key has the same digit are skipped on the device
        for label, keys in (("keys_below_2^32", k0 & 0xFFFFFFFF), ("all_keys_equal", torch.full_like(k0, 42))):
            def restore_low(keys=keys):
                k.copy_(keys)
                v.copy_(v0)
            ms = timed(fn, restore_low, 5, 1)
            assert torch.equal(keys[v.long()], k) and bool((k[1:] >= k[:-1]).all())
            extras[f"sort_by_key_u64_u32_{label}"] = {"value": round(n / float(np.median(ms)) / 1e6, 3), "unit": "Gkeys/s",
                                                      "ms": round(float(np.median(ms)), 4)}

    def extra_scan(dtype_name):
        if dtype_name == "i32":
            x = torch.randint(0, 16, (n,), dtype=torch.int32, device=dev, generator=gen(7))
            code = capi.I32
        else:
            x = torch.rand(n, dtype=torch.float32, device=dev, generator=gen(8)) * 2 - 1
            code = capi.F32
        out = torch.empty_like(x)
        for excl, label in ((0, "inclusive"), (1, "exclusive")):
            call = lambda t, nb: L.thrust_cdna4_scan(t, ctypes.byref(nb), code, capi.PLUS, excl,
                                                      ctypes.c_void_p(x.data_ptr()),
                                                      ctypes.c_void_p(out.data_ptr()), n, None, sp)
            tmp, nb = two_phase(call)
            tp = ctypes.c_void_p(tmp.data_ptr())
            fn = lambda: capi.check(call(tp, nb), "scan")
            ms = timed(fn, lambda: None, 10, 2)
            add_extra(f"{label}_scan_{dtype_name}", n, ms, 8.0 * n, "Gelem/s")
        if dtype_name == "i32":
            assert int(out[-1].item()) + int(x[-1].item()) == int(x.sum(dtype=torch.int64).item())

    def extra_scan_sweep():
        x = torch.randint(0, 16, (n,), dtype=torch.int32, device=dev, generator=gen(7))
        out = torch.empty_like(x)
        sweep = {}
        for lg in range(20, args.log2n + 1, 2):
            m = 1 << lg
            call = lambda t, nb: L.thrust_cdna4_scan(t, ctypes.byref(nb), capi.I32, capi.PLUS, 0,
                                                      ctypes.c_void_p(x.data_ptr()),
                                                      ctypes.c_void_p(out.data_ptr()), m, None, sp)
            tmp, nb = two_phase(call)
            tp = ctypes.c_void_p(tmp.data_ptr())
            ms = timed(lambda: capi.check(call(tp, nb), "scan"), lambda: None, 10, 2)
            sweep[f"2^{lg}"] = round(m / float(np.median(ms)) / 1e6, 2)
        extras["inclusive_scan_i32_sweep_gelem_per_s"] = sweep

    def extra_narrow():
        # 1- and 2-byte elements: the scan keeps them packed in registers, and one-byte keys without
        # values are sorted by histogram and fill (no key moves: 2 bytes of traffic per key)
        for tname, tdt, code in (("i8", torch.int8, capi.I8), ("i16", torch.int16, capi.I16)):
            x = torch.randint(-3, 4, (n,), dtype=tdt, device=dev, generator=gen(31))
            out = torch.empty_like(x)
            call = lambda t, nb: L.thrust_cdna4_scan(t, ctypes.byref(nb), code, capi.PLUS, 0, ctypes.c_void_p(x.data_ptr()),
                                                      ctypes.c_void_p(out.data_ptr()), n, None, sp)
            tmp, nb = two_phase(call)
            tp = ctypes.c_void_p(tmp.data_ptr())
            ms = timed(lambda: capi.check(call(tp, nb), "scan"), lambda: None, 10, 2)
            assert torch.equal(out[-1000:], torch.cumsum(x.to(torch.int32), 0, dtype=torch.int32)[-1000:].to(tdt))
            add_extra(f"inclusive_scan_{tname}", n, ms, 2.0 * x.element_size() * n, "Gelem/s")
            del x, out
        src = torch.randint(0, 256, (n,), dtype=torch.uint8, device=dev, generator=gen(32))
        k = torch.empty_like(src)
        call = lambda t, nb: L.thrust_cdna4_sort_keys(t, ctypes.byref(nb), capi.U8, ctypes.c_void_p(k.data_ptr()), n, 0, sp)
        tmp, nb = two_phase(call)
        tp = ctypes.c_void_p(tmp.data_ptr())
        ms = timed(lambda: capi.check(call(tp, nb), "sort_keys"), lambda: k.copy_(src), 10, 2)
        assert torch.equal(torch.bincount(k.to(torch.int64), minlength=256), torch.bincount(src.to(torch.int64), minlength=256))
        assert bool((k[1:] >= k[:-1]).all())
        add_extra("sort_u8_keys", n, ms, 2.0 * n, "Gkeys/s")

    def extra_rbk(mean):
        if mean == 1:
            keys = torch.arange(n, dtype=torch.int32, device=dev)
        else:
            # run ids with geometric run lengths of the given mean: a head with probability 1/mean
            heads = torch.rand(n, device=dev, generator=gen(20 + mean)) < (1.0 / mean)
            keys = torch.cumsum(heads.to(torch.int32), 0, dtype=torch.int32)
            del heads
        vals = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device=dev, generator=gen(9))
        ko = torch.empty_like(keys)
        vo = torch.empty_like(vals)
        nr = torch.zeros(1, dtype=torch.int64, device=dev)
        call = lambda t, nb: L.thrust_cdna4_reduce_by_key(
            t, ctypes.byref(nb), capi.I32, capi.I32, capi.PLUS, ctypes.c_void_p(keys.data_ptr()),
            ctypes.c_void_p(vals.data_ptr()), ctypes.c_void_p(ko.data_ptr()), ctypes.c_void_p(vo.data_ptr()),
            ctypes.c_void_p(nr.data_ptr()), n, sp)
        tmp, nb = two_phase(call)
        tp = ctypes.c_void_p(tmp.data_ptr())
        ms = timed(lambda: capi.check(call(tp, nb), "reduce_by_key"), lambda: None, 10, 2)
        r = int(nr.item())
        assert int(vo[:r].sum(dtype=torch.int64).item()) == int(vals.sum(dtype=torch.int64).item())
        add_extra(f"reduce_by_key_i32_mean{mean}", n, ms, 8.0 * n + 8.0 * r, "Gelem/s")
        extras[f"reduce_by_key_i32_mean{mean}"]["runs"] = r

    def extra_sbk(mean):
        # inclusive_scan_by_key with plus: int32 keys (geometric run lengths), int32 values
        heads = torch.rand(n, device=dev, generator=gen(20 + mean)) < (1.0 / mean)
        keys = torch.cumsum(heads.to(torch.int32), 0, dtype=torch.int32)
        del heads
        vals = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device=dev, generator=gen(9))
        out = torch.empty_like(vals)
        call = lambda t, nb: L.thrust_cdna4_scan_by_key(
            t, ctypes.byref(nb), capi.I32, capi.I32, capi.PLUS, 0, ctypes.c_void_p(keys.data_ptr()),
            ctypes.c_void_p(vals.data_ptr()), ctypes.c_void_p(out.data_ptr()), n, None, sp)
        tmp, nb = two_phase(call)
        tp = ctypes.c_void_p(tmp.data_ptr())
        ms = timed(lambda: capi.check(call(tp, nb), "scan_by_key"), lambda: None, 10, 2)
        # the last element of every run is the run's sum: together they add up to the total
        last = torch.ones(n, dtype=torch.bool, device=dev)
        last[:-1] = keys[1:] != keys[:-1]
        assert int(out[last].sum(dtype=torch.int64).item()) == int(vals.sum(dtype=torch.int64).item())
        add_extra(f"inclusive_scan_by_key_i32_mean{mean}", n, ms, 12.0 * n, "Gelem/s")

    def extra_hist():
        m = 1 << min(30, args.log2n + 2)
        s = torch.randint(0, 256, (m,), dtype=torch.uint8, device=dev, generator=gen(11))
        counts = torch.empty(4096, dtype=torch.int32, device=dev)
        for bins in (256, 4096):
            call = lambda t, nb: L.thrust_cdna4_histogram_even(
                t, ctypes.byref(nb), capi.U8, ctypes.c_void_p(s.data_ptr()), m,
                ctypes.c_void_p(counts.data_ptr()), bins, 0.0, 256.0, sp)
            tmp, nb = two_phase(call)
            tp = ctypes.c_void_p(tmp.data_ptr())
            ms = timed(lambda: capi.check(call(tp, nb), "histogram"), lambda: None, 5, 1)
            assert int(counts[:bins].sum().item()) == m
            add_extra(f"histogram_u8_{bins}bins", m, ms, 1.0 * m, "Gsamples/s")
        del s
        # Zipf(1.1) ranks over 4096 values as fp32
        w = 1.0 / torch.arange(1, 4097, dtype=torch.float64, device=dev) ** 1.1
        cdf = torch.cumsum(w / w.sum(), 0).to(torch.float32)
        u = torch.rand(m, dtype=torch.float32, device=dev, generator=gen(12))
        f = torch.searchsorted(cdf, u).clamp_(max=4095).to(torch.float32)
        for bins in (256, 4096):
            call = lambda t, nb: L.thrust_cdna4_histogram_even(
                t, ctypes.byref(nb), capi.F32, ctypes.c_void_p(f.data_ptr()), m,
                ctypes.c_void_p(counts.data_ptr()), bins, 0.0, 4096.0, sp)
            tmp, nb = two_phase(call)
            tp = ctypes.c_void_p(tmp.data_ptr())
            ms = timed(lambda: capi.check(call(tp, nb), "histogram"), lambda: None, 5, 1)
            assert int(counts[:bins].sum().item()) == m
            add_extra(f"histogram_f32_zipf_{bins}bins", m, ms, 4.0 * m, "Gsamples/s")

    def extra_copy_ceiling():
        a = torch.empty(n, dtype=torch.int32, device=dev)
        b = torch.empty_like(a)
        ms = timed(lambda: b.copy_(a), lambda: None, 10, 2)
        extras["device_copy_ceiling_GBs"] = round(8.0 * n / float(np.median(ms)) / 1e6, 1)
        # the library's own device-to-device copy (one 16-byte access per thread)
        nbytes = ctypes.c_size_t(4 * n)
        ms = timed(lambda: capi.check(L.thrust_cdna4_memcpy_dtod(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(a.data_ptr()),
                                                                  nbytes, sp), "memcpy_dtod"), lambda: None, 10, 2)
        extras["library_copy_GBs"] = round(8.0 * n / float(np.median(ms)) / 1e6, 1)

    def extra_merge_sort():
        # comparison sort with a user comparator: kernel templates, so a C++ binary built by hipcc
        # (tests/cpp/bench_merge_sort.cpp) measures it; 2^26 keys
        import subprocess
        exe = os.path.join(ROOT, "tests", "cpp", "build", "bench_merge_sort")
        if not os.path.exists(exe):
            return
        r = subprocess.run([exe, "26"], capture_output=True, text=True, timeout=300)
        if r.returncode == 0:
            extras.update(json.loads(r.stdout.strip().splitlines()[-1]))

    def extra_generic():
        # transform / reduce with user functors (kernel templates): tests/cpp/bench_generic.cpp, 2^28 floats
        import subprocess
        exe = os.path.join(ROOT, "tests", "cpp", "build", "bench_generic")
        if not os.path.exists(exe):
            return
        r = subprocess.run([exe, str(args.log2n)], capture_output=True, text=True, timeout=300)
        if r.returncode == 0:
            extras.update(json.loads(r.stdout.strip().splitlines()[-1]))

    def extra_select():
        # copy_if / unique / unique_by_key with user predicates (kernel templates): tests/cpp/bench_select.cpp
        import subprocess
        exe = os.path.join(ROOT, "tests", "cpp", "build", "bench_select")
        if not os.path.exists(exe):
            return
        r = subprocess.run([exe, str(args.log2n)], capture_output=True, text=True, timeout=300)
        if r.returncode == 0:
            extras.update(json.loads(r.stdout.strip().splitlines()[-1]))

    def extra_api():
        # what a caller of thrust::sort / thrust::inclusive_scan sees: header dispatch, pool,
        # launches and synchronisation inside the timed call, the first call of a process on its
        # own, and the user-operator engine (tests/cpp/bench_api.cpp)
        import subprocess
        exe = os.path.join(ROOT, "tests", "cpp", "build", "bench_api")
        if not os.path.exists(exe):
            return
        r = subprocess.run([exe, str(args.log2n)], capture_output=True, text=True, timeout=600)
        if r.returncode == 0:
            extras.update(json.loads(r.stdout.strip().splitlines()[-1]))
        else:
            extras["api_error"] = r.stderr[-300:]

    all_extras = {
        "api": extra_api,
        "generic": extra_generic,
        "select": extra_select,
        "merge_sort": extra_merge_sort,
        "sort_by_key": extra_sort_pairs,
        "scan_i32": lambda: extra_scan("i32"),
        "scan_f32": lambda: extra_scan("f32"),
        "scan_sweep": extra_scan_sweep,
        "narrow": extra_narrow,
        "rbk1": lambda: extra_rbk(1),
        "rbk8": lambda: extra_rbk(8),
        "rbk512": lambda: extra_rbk(512),
        "sbk8": lambda: extra_sbk(8),
        "hist": extra_hist,
        "copy": extra_copy_ceiling,
    }
    if not args.no_extras:
        for name, f in all_extras.items():
            if args.only and name != args.only:
                continue
            f()
            torch.cuda.empty_cache()

    # ------------------------------------------------------------------ CPU baseline
    cpu = None
    if not args.no_cpu:
        import oracle
        threads = oracle.omp_max_threads()
        m = n  # the whole GPU workload: a few seconds per repetition on 16 cores
        ks = np.random.default_rng(1337).integers(0, 2**32, m, dtype=np.uint64).astype(np.uint32)
        best = None
        for _ in range(3):
            k = ks.copy()
            t0 = time.perf_counter()
            oracle.omp_sort(k, None, threads)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        assert (k[1:] >= k[:-1]).all()
        cpu = {
            "value": round(m / best / 1e9, 4), "unit": "Gkeys/s", "cores": threads, "kind": "port",
            "sample": f"2^{args.log2n} uniform uint32 keys (the whole GPU workload), best of 3; oracle "
                      f"restatement of the reference OpenMP sort (per-thread radix sort with the reference's "
                      f"digit widths, 4 bits for these tiles, + pairwise merges)",
        }

        # the other algorithms of the path: the scalar oracle (the reference's sequential loops
        # restated, 1 core) on a 2^26-element sample of the workloads of the extras above
        if not args.no_extras and not args.only:
            m = min(n, 1 << 26)
            rng = np.random.default_rng(7)

            def best_of(f, reps=3):
                best = None
                for _ in range(reps):
                    t0 = time.perf_counter()
                    f()
                    dt = time.perf_counter() - t0
                    best = dt if best is None else min(best, dt)
                return best

            xi = rng.integers(0, 16, m, dtype=np.int32)
            keys8 = np.cumsum(rng.random(m) < 1.0 / 8, dtype=np.int32)
            vals = rng.integers(-1000, 1001, m, dtype=np.int32)
            zipf_w = 1.0 / np.arange(1, 4097, dtype=np.float64) ** 1.1
            samples = np.searchsorted(np.cumsum(zipf_w / zipf_w.sum()), rng.random(m)).clip(max=4095).astype(np.float32)
            extras["cpu_baselines"] = {
                "kind": "port", "cores": 1, "sample": "2^%d elements, best of 3" % int(np.log2(m)),
                "inclusive_scan_i32_gelem_per_s": round(m / best_of(lambda: oracle.scan(xi)) / 1e9, 4),
                "reduce_by_key_i32_mean8_gelem_per_s": round(m / best_of(lambda: oracle.reduce_by_key(keys8, vals)) / 1e9, 4),
                "inclusive_scan_by_key_i32_mean8_gelem_per_s": round(m / best_of(lambda: oracle.scan_by_key(keys8, vals)) / 1e9, 4),
                "histogram_f32_zipf_256bins_gsamples_per_s": round(m / best_of(lambda: oracle.histogram_even(samples, 256, 0.0, 4096.0)) / 1e9, 4),
            }

    out = {
        "metric": "thrust::sort throughput, 2^%d uint32 keys" % args.log2n,
        "value": round(gkeys, 3),
        "unit": "Gkeys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": "thrust::sort of 2^%d uniform uint32 keys (seed 1337), ascending, "
                               "in place through thrust_cdna4_sort_keys" % args.log2n,
                   "n": n, "algorithmic_bytes_per_key": 36,
                   "whole_sort_roofline_frac": round(sort_bytes / ms_per_step / 1e6 / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "kernel": "onesweep_kernel<uint32, keys only>",
                     "achieved": round(onesweep_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(onesweep_gbs / HBM_PEAK_GBS, 4),
                     # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE (x2.000) + WRITE_SIZE (x1.000),
                     # scale factors from a plain 1 GiB copy; summary under profiles/ (n = 2^28 only)
                     "traffic": ONESWEEP_U32_TRAFFIC_BYTES if args.log2n == 28 else None,
                     "avg_launch_ms": round(onesweep_ms, 4), "launches_timed": onesweep_launches,
                     "algorithmic_bytes_per_launch": onesweep_bytes},
        "cpu_baseline": cpu,
        "extras": extras,
        "wall_s": round(time.time() - t_wall0, 1),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
