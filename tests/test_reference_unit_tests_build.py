"""The reference's own unit tests (testing/*.cu, with its harness testing/unittest/) are compiled
unchanged against include/ — syntax and semantic analysis of the host and the device pass, no code
generation.  tests/golden/reference_unit_tests.json lists the files that compile; each must still
compile, and none may take a header from another Thrust on the include path.  Needs the reference
tree and hipcc; skipped where either is missing."""
import json
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_TESTING = "/root/reference/testing"
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

with open(os.path.join(ROOT, "tests", "golden", "reference_unit_tests.json")) as f:
    GOLDEN = json.load(f)


def _check(name):
    cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only", "-w", "-H", "-ferror-limit=3",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "tests", "shim"), "-I" + REF_TESTING, os.path.join(REF_TESTING, name + ".cu")]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    foreign = sorted({ln.split()[-1] for ln in p.stderr.splitlines()
                      if ln.startswith(".") and "/include/thrust/" in ln and not ln.split()[-1].startswith((ROOT, REF_TESTING))})
    errors = [ln for ln in p.stderr.splitlines() if " error: " in ln][:3]
    return name, p.returncode, errors, foreign


@pytest.mark.skipif(not os.path.isdir(REF_TESTING) or not os.path.exists(HIPCC), reason="needs the reference tree and hipcc")
def test_reference_unit_tests_compile_unchanged():
    present = {f[:-3] for f in os.listdir(REF_TESTING) if f.endswith(".cu")}
    assert set(GOLDEN["compiling"]) | set(GOLDEN["not_compiling"]) == present
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(_check, GOLDEN["compiling"]))
    broken = {name: errors for name, rc, errors, _ in results if rc != 0}
    assert not broken, broken
    leaked = {name: foreign for name, _, _, foreign in results if foreign}
    assert not leaked, leaked


# Reference test files whose host-vector variants (test names ending in "Host") run here on the
# CPU; the few of those that move data to or from a device vector need a device and are left out.
CORE = ["sort", "stable_sort", "sort_by_key", "stable_sort_by_key", "scan_by_key.inclusive", "scan_by_key.exclusive",
        "reduce_by_key", "reduce", "vector", "vector_insert", "vector_manipulation", "unique", "unique_by_key", "merge",
        "set_union", "partition_point", "remove", "replace", "transform", "gather", "scatter", "tuple", "pair"]
NEEDS_A_DEVICE = {"TestVectorAssignFromDeviceVectorHost", "TestVectorToAndFromDeviceVectorHost", "TestTupleSwap", "TestTupleTie",
                  "TestPairSwap"}
DEVICE_FREE_FILES = {"tuple", "pair"}  # every other test of these files runs on the CPU


@pytest.mark.skipif(not os.path.isdir(REF_TESTING) or not os.path.exists(HIPCC), reason="needs the reference tree and hipcc")
def test_reference_host_vector_tests_pass_on_the_cpu():
    """The reference's unit tests, built unchanged by `make -C oracle ref_tests`, run their
    host-vector variants: the host system of this header layer (thrust::host_vector, the sequential
    algorithm forms, tuple, pair, dispatch on host iterators) against the reference's own checks."""
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "ref_tests", "-j8"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    ran = 0
    for name in CORE:
        exe = os.path.join(ROOT, "oracle", "_ref", "testing", name)
        listed = subprocess.run([exe, "--list"], stdout=subprocess.PIPE, text=True).stdout.split()
        names = [t for t in listed if t not in NEEDS_A_DEVICE] if name in DEVICE_FREE_FILES else [
            t for t in listed if (t.endswith("Host") or t.endswith("<thrust::host_vector>")) and t not in NEEDS_A_DEVICE]
        if not names:  # a file whose tests all use the device
            continue
        p = subprocess.run([exe] + names, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
        assert p.returncode == 0 and "0 failures, 0 known failures, 0 errors" in p.stdout, name + "\n" + p.stdout[-3000:]
        ran += len(names)
    assert ran >= 80, ran
