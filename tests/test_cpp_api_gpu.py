"""Runs the C++ API tests (tests/cpp/*.cpp) on the GPU.  All but one are plain g++ translation
units that use thrust::device_vector, thrust::sort, thrust::inclusive_scan,
thrust::reduce_by_key ... from include/thrust and link only against libthrust_cdna4.so; each
mirrors one of the reference's own test files and compares host and device results."""
import os
import subprocess

import pytest

from conftest import ROOT

BIN_DIR = os.path.join(ROOT, "tests", "cpp", "build")
# test_scan_generic, test_merge_sort, test_generic and test_select instantiate kernel templates with user functors and are compiled by hipcc
BINARIES = ["test_system_dir", "test_dispatch", "test_algorithms", "test_complex", "test_merge_set", "test_memory", "test_sort", "test_scan", "test_by_key", "test_system", "test_host_vector", "test_scan_generic", "test_merge_sort", "test_generic", "test_select", "test_partition", "test_iterators", "test_async", "test_mr", "test_api_surface", "test_seq"]


@pytest.mark.gpu
@pytest.mark.parametrize("name", BINARIES)
def test_cpp_api(name):
    path = os.path.join(BIN_DIR, name)
    if not os.path.exists(path):  # normally prebuilt by __graft_entry__.build()
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), f"build/{name}"], check=True)
    r = subprocess.run([path], capture_output=True, text=True, timeout=600)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-2000:]
    assert "0 failed" in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["test_sort", "test_scan", "test_by_key", "test_system"])
def test_cpp_api_host_side_under_sanitizers(name):
    """The host-compiled tests built with -fsanitize=address,undefined: headers, dispatch, vectors
    and the calls into the library, checked for out-of-bounds accesses, use after free and
    undefined behaviour on the host side (leaks of the HIP runtime itself are not ours to report)."""
    path = os.path.join(BIN_DIR, "san", name)
    if not os.path.exists(path):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), f"build/san/{name}"], check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([path], capture_output=True, text=True, timeout=900, env=env)
    print(r.stdout[-3000:])
    print(r.stderr[-3000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "0 failed" in r.stdout
