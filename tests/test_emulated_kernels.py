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


@pytest.fixture(scope="module")
def emulated_library():
    r = subprocess.run(["make", "-C", EMU_DIR, "-j8"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert os.path.exists(EMU_LIB)
    return EMU_LIB


def run_session(files, resident="1", deselect=(), extra=()):
    env = dict(os.environ, THRUST_CDNA4_EMULATED="1", THRUST_CDNA4_EMULATED_RESIDENT=resident)
    env.pop("THRUST_CDNA4_LIB", None)
    cmd = [sys.executable, "-m", "pytest", "-m", "gpu", "-q", "-x", "-p", "no:cacheprovider", "-n", WORKERS,
           "--timeout", "900", *files, *extra]
    if not ALL:
        for d in deselect:
            cmd += ["--deselect", d]
    r = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True)
    tail = r.stdout[-6000:] + r.stderr[-2000:]
    assert r.returncode == 0, tail
    last = [line for line in r.stdout.splitlines() if " passed" in line]
    assert last and "failed" not in last[-1], tail
    return last[-1]


def test_scans_by_key_and_histogram_one_workgroup_at_a_time(emulated_library):
    print(run_session(["tests/test_scan_gpu.py", "tests/test_bykey_gpu.py", "tests/test_histogram_gpu.py",
                       "tests/test_zz_no_alloc.py"], deselect=SLOW))


def test_sorts_one_workgroup_at_a_time(emulated_library):
    print(run_session(["tests/test_sort_gpu.py", "tests/test_random_gpu.py"], deselect=SLOW))


@pytest.mark.parametrize("resident", ["6:11", "16:5", "3:77"] if ALL else ["6:11"])
def test_look_back_with_several_workgroups_in_flight(emulated_library, resident):
    """Tiles meet predecessors that have published a partial result or nothing yet; a sort whose
    look-back is made to give up reports it (the status word, the error, the latch to plain tickets)."""
    print(run_session(["tests/test_scan_gpu.py", "tests/test_bykey_gpu.py", "tests/test_random_gpu.py",
                       "tests/test_sort_timeout_gpu.py"], resident=resident, deselect=SLOW))
