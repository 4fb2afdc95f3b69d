"""The GPU parity tests, run WITHOUT a GPU: the kernel sources of thrust_amd/csrc are compiled for
the host against a stand-in HIP header and executed lane by lane by the lockstep emulator of
tests/emu (wavefronts of 64 lanes, DPP / ds_bpermute / readlane / ballot, LDS, workgroup barriers,
atomics served in lane order, several workgroups in flight with seeded interleavings).  The same
test files, the same oracle, the same C ABI — what changes is who executes the kernels.

This checks what the kernels COMPUTE (indexing, tile edges, the order in which partial results are
combined, the look-back protocol under many interleavings, status reporting) on every machine, and
stands in for nothing: performance, memory ordering, register and LDS budgets and the hardware's
own behaviour are only seen by the tests marked gpu when they run on the device.

Each test below starts one pytest session of its own with THRUST_CDNA4_EMULATED=1 (tests/conftest.py
then serves `thrust_amd` from the emulated library and CPU tensors).  The default selection is sized
for a few minutes on 8 cores; THRUST_CDNA4_EMULATE_ALL=1 adds the tests that take minutes each.
"""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU_DIR = os.path.join(ROOT, "tests", "emu")
EMU_LIB = os.path.join(EMU_DIR, "build", "libthrust_cdna4_emu.so")
WORKERS = str(max(1, min(6, (os.cpu_count() or 2) - 1)))

ALL = os.environ.get("THRUST_CDNA4_EMULATE_ALL") == "1"

# minutes each under emulation (inputs of 2^21 and more, chosen to reach the large-tile kernels)
SLOW = [
    "tests/test_sort_gpu.py::test_sort_skips_places_where_all_keys_agree",
    "tests/test_sort_gpu.py::test_sort_pairs_large_tiles_stability",
    "tests/test_sort_gpu.py::test_sort_keys_large_tiles_all_types",
    "tests/test_sort_gpu.py::test_sort_one_byte_keys_by_counting",
    "tests/test_sort_gpu.py::test_sort_unaligned_views_and_repeat_determinism",
    "tests/test_zz_no_alloc.py::test_float_and_in_place_and_large",
]


# C++ API tests (tests/cpp) that the default run leaves out: minutes of emulation each, or inputs of
# 2^30 items and more that only a device gets through (the latter are left out in every mode)
CPP_NEVER = ["BigIndexes"]
CPP_SLOW = ["TestStableSortRepeatable", "TestCopyIfLarge", "TestVectorSearch", "TestFindMismatchLadder", "TestShuffle",
            "TestStablePartitionLarge", "TestStableSortByKey<", "TestAsyncSort",
            # of a typed test the default run keeps the int / int32_t instance
            "<int8_t>", "<uint8_t>", "<int16_t>", "<uint16_t>", "<uint32_t>", "<int64_t>", "<uint64_t>", "<float>",
            "<double>"]
CPP_TESTS = ["test_sort", "test_scan", "test_by_key", "test_host_vector", "test_seq", "test_system_dir",
             "test_dispatch", "test_complex", "test_memory", "test_merge_set", "test_algorithms",
             "test_scan_generic", "test_merge_sort", "test_generic", "test_select", "test_partition",
             "test_iterators", "test_async", "test_mr", "test_api_surface", "test_system"]


@pytest.fixture(scope="module")
def emulated_library():
    r = subprocess.run(["make", "-C", EMU_DIR, "-j8"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert os.path.exists(EMU_LIB)
    return EMU_LIB


def run_session(files, resident="1", deselect=(), extra=(), guard=False):
    env = dict(os.environ, THRUST_CDNA4_EMULATED="1", THRUST_CDNA4_EMULATED_RESIDENT=resident,
               THRUST_CDNA4_EMULATED_GUARD="1" if guard else "0")
    env.pop("THRUST_CDNA4_LIB", None)
    cmd = [sys.executable, "-X", "faulthandler", "-m", "pytest", "-m", "gpu", "-q", "-x", "-p", "no:cacheprovider", *files, *extra]
    try:  # workers and a per-test time limit where the plugins are there
        import xdist  # noqa: F401
        cmd += ["-n", WORKERS]
    except ImportError:
        pass
    try:
        import pytest_timeout  # noqa: F401
        cmd += ["--timeout", "900"]
    except ImportError:
        pass
    if not ALL:
        for d in deselect:
            cmd += ["--deselect", d]
    r = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True)
    tail = r.stdout[-6000:] + r.stderr[-2000:]
    assert r.returncode == 0, tail
    last = [line for line in r.stdout.splitlines() if " passed" in line]
    assert last and "failed" not in last[-1], tail
    return last[-1]


def test_one_workgroup_at_a_time_and_no_byte_outside_the_ranges(emulated_library):
    """Every "device" buffer of this session (inputs, outputs, temporary storage) ends where an
    inaccessible page begins: a kernel that reads or writes past the end of a range it was given
    ends the session with a segmentation fault.  Workgroups run one after the other."""
    print(run_session(["tests/test_sort_gpu.py", "tests/test_random_gpu.py", "tests/test_histogram_gpu.py", "tests/test_zz_no_alloc.py",
                       "tests/test_scan_gpu.py", "tests/test_bykey_gpu.py"], deselect=SLOW, guard=True))


@pytest.mark.parametrize("resident", ["6:11", "16:5", "3:77"] if ALL else ["6:11"])
def test_look_back_with_several_workgroups_in_flight(emulated_library, resident):
    """Tiles meet predecessors that have published a partial result or nothing yet; a sort whose
    look-back is made to give up reports it (the status word, the error, the latch to plain tickets)."""
    files = ["tests/test_scan_gpu.py", "tests/test_bykey_gpu.py", "tests/test_random_gpu.py", "tests/test_sort_timeout_gpu.py",
             "tests/test_dirty_temp_gpu.py"]  # (dirty descriptors only matter to a tile that runs before its predecessor is done)
    if ALL:  # (buffers aligned as an allocator aligns them; the default run has the sorts in the guarded session only)
        files += ["tests/test_sort_gpu.py", "tests/test_histogram_gpu.py", "tests/test_zz_no_alloc.py"]
    print(run_session(files, resident=resident, deselect=SLOW))


def test_cpp_api_tests_on_the_emulated_library(emulated_library):
    """The header layer's own kernels (user operators, merge sort, select and partition, merge and
    set operations, thrust::seq inside kernels) through the C++ API tests of tests/cpp, built for
    the host by tests/emu/Makefile."""
    from concurrent.futures import ThreadPoolExecutor

    env = dict(os.environ, THRUST_CDNA4_TEST_SKIP=",".join(CPP_NEVER + ([] if ALL else CPP_SLOW)))

    def run(name):
        r = subprocess.run([os.path.join(EMU_DIR, "build", "cpp", name)], env=env, capture_output=True, text=True,
                           timeout=1800)
        return name, r.returncode, r.stdout[-3000:] + r.stderr[-1000:]

    with ThreadPoolExecutor(int(WORKERS)) as pool:
        results = list(pool.map(run, CPP_TESTS))
    failed = [(name, out) for name, rc, out in results if rc != 0 or "0 failed" not in out]
    assert not failed, failed
    ran = sum(int(out.strip().splitlines()[-1].split()[0]) for _, _, out in results)
    assert ran > (380 if ALL else 200), ran


REF_TESTING = "/root/reference/testing"
# The reference's unit test files of the hot path and its nearest callers (the default set of
# tests/emu/Makefile's ref_tests); THRUST_CDNA4_EMULATE_ALL=1 runs every file that compiles.
REF_DEFAULT = ["sort", "sort_by_key", "stable_sort", "stable_sort_by_key", "sort_variable_bits", "sort_by_key_variable_bits",
               "stable_sort_large", "stable_sort_by_key_large_keys", "stable_sort_by_key_large_values",
               "stable_sort_by_key_large_keys_and_values", "sort_permutation_iterator", "scan", "copy", "scan_by_key.inclusive",
               "scan_by_key.exclusive", "reduce_by_key", "transform_scan", "pair_scan", "pair_scan_by_key", "pair_sort",
               "pair_sort_by_key", "tuple_scan", "tuple_sort", "zip_iterator_scan", "zip_iterator_sort", "zip_iterator_sort_by_key",
               "zip_iterator_reduce_by_key", "transform_output_iterator_reduce_by_key"]
# not run under emulation, with the reason
REF_FILES_LEFT_OUT = {
    "unittest_static_assert": "throws a C++ exception from device code, which on the emulator is a fiber with no frame to catch it",
}
REF_TESTS_LEFT_OUT = {
    "WithBigIndexes": "2^30 to 2^33 elements: hours of emulation",
}


@pytest.mark.skipif(not os.path.isdir(REF_TESTING), reason="needs the reference tree")
def test_reference_unit_tests_on_the_emulated_library(emulated_library):
    """The reference's own unit tests, compiled unchanged (tests/emu/Makefile, ref_tests) and run
    with their device_vector variants executing on the emulated library: its checks, its sizes, its
    harness.  Every test of every file must pass; what is left out is listed above with the reason."""
    import json
    from concurrent.futures import ThreadPoolExecutor

    with open(os.path.join(ROOT, "tests", "golden", "reference_unit_tests.json")) as f:
        compiling = json.load(f)["compiling"]
    names = [n for n in (compiling if ALL else REF_DEFAULT) if n not in REF_FILES_LEFT_OUT]
    assert set(REF_DEFAULT) <= set(compiling)
    r = subprocess.run(["make", "-C", EMU_DIR, "-j8", "ref_tests", "REF_TESTS=" + " ".join(names)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]

    def run(name):
        exe = os.path.join(EMU_DIR, "build", "ref", name)
        listed = subprocess.run([exe, "--list"], capture_output=True, text=True).stdout.split()
        tests = [t for t in listed if not any(skip in t for skip in REF_TESTS_LEFT_OUT)]
        if not tests:
            return name, 0, 0, ""
        p = subprocess.run([exe] + tests, capture_output=True, text=True, timeout=3000)
        # (a "known failure" is the reference's own marking of a test it expects to fail)
        ok = p.returncode == 0 and re.search(r"Totals: 0 failures, \d+ known failures, 0 errors", p.stdout) is not None
        return name, len(tests), ok, p.stdout[-2500:] + p.stderr[-500:]

    with ThreadPoolExecutor(int(WORKERS)) as pool:
        results = list(pool.map(run, names))
    failed = [(name, out) for name, count, ok, out in results if count and not ok]
    assert not failed, failed
    ran = sum(count for _, count, _, _ in results)
    assert ran >= (1200 if ALL else 110), ran
    print(f"{ran} tests of {len(names)} reference files")


@pytest.mark.skipif(not ALL, reason="builds the library once more under ThreadSanitizer: THRUST_CDNA4_EMULATE_ALL=1")
def test_no_data_race_between_wavefronts(emulated_library):
    """The race-detecting build (tests/emu/Makefile, tsan): ThreadSanitizer sees every wavefront as a
    thread, workgroup barriers (and the ends of a launch) as the only ordering between them, and the
    workgroups in flight as threads of the process.  A missing barrier around an LDS exchange, or one
    workgroup reading what another is still writing, is a reported data race.  The self-test shows that
    such races ARE reported; then the scan, by-key and sort tests of tests/cpp must run clean."""
    r = subprocess.run(["make", "-C", EMU_DIR, "-j8", "tsan"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    tsan = os.path.join(EMU_DIR, "build", "tsan")

    def reports(args, resident="1"):
        env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0", THRUST_CDNA4_EMULATED_RESIDENT=resident)
        p = subprocess.run([os.path.join(tsan, "selftest_race")] + args, env=env, capture_output=True, text=True, timeout=300)
        return (p.stdout + p.stderr).count("WARNING: ThreadSanitizer: data race")

    assert reports(["with_barrier"]) == 0
    assert reports(["without_barrier"]) >= 1
    assert reports(["global"]) >= 1
    assert sum(reports(["across_workgroups"], f"2:{seed}") for seed in range(1, 9)) >= 1

    from concurrent.futures import ThreadPoolExecutor

    typed = ("BigIndexes,Repeatable,Large,VectorSearch,FindMismatch,Shuffle,"
             "<int8_t>,<uint8_t>,<int16_t>,<uint16_t>,<uint32_t>,<uint64_t>,<float>,<short>")

    def clean(case):
        name, resident = case
        env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1", THRUST_CDNA4_EMULATED_RESIDENT=resident, THRUST_CDNA4_TEST_SKIP=typed)
        p = subprocess.run([os.path.join(tsan, name)], env=env, capture_output=True, text=True, timeout=3000)
        out = p.stdout + p.stderr
        return case, p.returncode == 0 and "ThreadSanitizer" not in out and ", 0 failed" in out, out[-4000:]

    # the hot path's kernels, then the header layer's own (user operators, select, partition, merge sort, merge / set operations)
    names = ["test_scan", "test_by_key", "test_sort", "test_scan_generic", "test_select", "test_partition", "test_merge_sort",
             "test_merge_set", "test_generic", "test_algorithms", "test_seq"]
    cases = [(name, resident) for resident in ("1", "4:9") for name in names]
    with ThreadPoolExecutor(int(WORKERS)) as pool:
        bad = [(case, out) for case, ok, out in pool.map(clean, cases) if not ok]
    assert not bad, bad


@pytest.mark.skipif(not os.path.isdir("/root/reference/examples"), reason="needs the reference tree")
def test_reference_examples_on_the_emulated_library(emulated_library):
    """The reference's 51 example programs, compiled unchanged (tests/emu/Makefile, ref_examples): their
    output must satisfy the golden outputs the reference keeps for them, as it must on the GPU
    (tests/test_reference_examples.py, whose matcher and golden data this uses)."""
    from concurrent.futures import ThreadPoolExecutor

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from test_reference_examples import EXAMPLES, GOLDEN, filecheck

    r = subprocess.run(["make", "-C", EMU_DIR, "-j8", "ref_examples"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]

    def run(name):
        p = subprocess.run([os.path.join(EMU_DIR, "build", "examples", name)], capture_output=True, text=True, timeout=900)
        if p.returncode != 0:
            return name, "exit code %d\n%s" % (p.returncode, (p.stdout + p.stderr)[-1500:])
        return name, filecheck(p.stdout, GOLDEN[name]["checks"])

    with ThreadPoolExecutor(int(WORKERS)) as pool:
        problems = [(name, why) for name, why in pool.map(run, EXAMPLES) if why is not None]
    assert not problems, problems
    assert len(EXAMPLES) == 51
