"""CPU-only: user code written against the Thrust API surface builds with a plain host
compiler against include/thrust (no device compiler in the user's build), and the headers
refuse what the device system has no kernel for instead of falling back to the host."""
import os
import subprocess
import textwrap

from conftest import ROOT

INC = os.path.join(ROOT, "include")


def compile_snippet(tmp_path, body, extra=()):
    src = tmp_path / "t.cpp"
    src.write_text(textwrap.dedent(body))
    return subprocess.run(["g++", "-std=c++14", "-fsyntax-only", "-I", INC, *extra, str(src)],
                          capture_output=True, text=True)


def test_cpp_tests_compile():
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    for name in ["test_system_dir", "test_dispatch", "test_algorithms", "test_complex", "test_merge_set", "test_memory", "test_sort", "test_scan", "test_by_key", "test_system", "test_host_vector", "test_scan_generic", "test_merge_sort", "bench_merge_sort", "test_generic", "test_select", "bench_select", "test_partition", "test_iterators", "test_async", "test_mr", "test_api_surface", "test_seq",
                 "bench_generic", "bench_api"]:
        assert os.path.exists(os.path.join(ROOT, "tests", "cpp", "build", name))


def test_seq_algorithms_on_the_cpu():
    # thrust::seq on host ranges: the sequential sort (in place, by rotations), scans and
    # reduce_by_key that kernels call as well; the kernel half of the file runs on the GPU
    path = os.path.join(ROOT, "tests", "cpp", "build", "test_seq")
    r = subprocess.run([path, "Host"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "2 tests, 0 failed" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_oracle_runs_clean_under_the_sanitizers():
    # every entry point of the CPU oracle over small inputs of every type, operator and flag, built
    # with -fsanitize=address,undefined: the parity tests trust it as their reference
    r = subprocess.run(["make", "-B", "-C", os.path.join(ROOT, "oracle"), "selfcheck"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([os.path.join(ROOT, "oracle", "selfcheck")], capture_output=True, text=True,
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1"))
    assert r.returncode == 0 and "selfcheck: ok" in r.stdout, r.stdout[-2000:] + r.stderr[-3000:]


def test_host_compiled_tests_build_under_the_sanitizers():
    # the g++ translation units once more with -fsanitize=address,undefined (run on the GPU by
    # tests/test_cpp_api_gpu.py)
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "san"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    for name in ["test_sort", "test_scan", "test_by_key", "test_system", "test_host_vector"]:
        assert os.path.exists(os.path.join(ROOT, "tests", "cpp", "build", "san", name))


def test_host_vector_container_on_the_cpu():
    # thrust::host_vector is host code only: its tests run here, plain and under the sanitizers
    for sub in ("", "san"):
        path = os.path.join(ROOT, "tests", "cpp", "build", sub, "test_host_vector")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), os.path.join("build", sub, "test_host_vector")], check=True)
        r = subprocess.run([path], capture_output=True, text=True, timeout=300,
                           env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1"))
        assert r.returncode == 0 and "0 failed" in r.stdout, r.stdout[-2000:] + r.stderr[-3000:]


def test_existing_thrust_code_compiles_unchanged(tmp_path):
    r = compile_snippet(tmp_path, """
        #include <thrust/device_vector.h>
        #include <thrust/host_vector.h>
        #include <thrust/execution_policy.h>
        #include <thrust/sort.h>
        #include <thrust/scan.h>
        #include <thrust/reduce.h>
        #include <thrust/functional.h>
        int main() {
          thrust::host_vector<int> h(1000);
          thrust::device_vector<int> d = h, o(1000), k(1000), v(1000);
          thrust::sort(d.begin(), d.end());
          thrust::sort(thrust::device, d.begin(), d.end(), thrust::greater<int>());
          thrust::sort_by_key(d.begin(), d.end(), o.begin());
          thrust::inclusive_scan(thrust::device, d.begin(), d.end(), o.begin());
          thrust::exclusive_scan(d.begin(), d.end(), o.begin(), 0, thrust::plus<int>());
          thrust::inclusive_scan_by_key(d.begin(), d.end(), o.begin(), v.begin());
          auto e = thrust::reduce_by_key(d.begin(), d.end(), o.begin(), k.begin(), v.begin());
          return (int)(e.first - k.begin());
        }""")
    assert r.returncode == 0, r.stderr[-3000:]


def test_headers_shadow_any_other_thrust(tmp_path):
    # /opt/rocm/include also holds a <thrust/...>; with -I include first ours must win
    r = compile_snippet(tmp_path, """
        #include <thrust/version.h>
        #include <thrust/sort.h>
        static_assert(THRUST_CDNA4_VERSION >= 100, "resolved to a foreign thrust");
        int main() { return 0; }""", extra=("-isystem", "/opt/rocm/include"))
    assert r.returncode == 0, r.stderr[-3000:]


def test_unsupported_comparator_is_a_compile_error_not_a_host_fallback(tmp_path):
    r = compile_snippet(tmp_path, """
        #include <thrust/device_vector.h>
        #include <thrust/sort.h>
        struct by_mod3 { bool operator()(int a, int b) const { return a % 3 < b % 3; } };
        int main() { thrust::device_vector<int> d(10); thrust::sort(d.begin(), d.end(), by_mod3()); }""")
    assert r.returncode != 0
    assert "compile this translation unit with hipcc" in r.stderr


def test_custom_comparator_compiles_with_hipcc(tmp_path):
    # the same code builds when the device compiler can instantiate the comparison-sort kernels
    src = tmp_path / "t.cpp"
    src.write_text(textwrap.dedent("""
        #include <thrust/device_vector.h>
        #include <thrust/sort.h>
        struct by_mod3 { __host__ __device__ bool operator()(int a, int b) const { return a % 3 < b % 3; } };
        int main() { thrust::device_vector<int> d(10), v(10); thrust::sort(d.begin(), d.end(), by_mod3());
                     thrust::stable_sort_by_key(d.begin(), d.end(), v.begin(), by_mod3()); }"""))
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only",
                        "-I", INC, str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_exclusive_scan_accumulates_in_the_type_of_init(tmp_path):
    # thrust/system/cuda/detail/scan.h:142-154: the accumulator has init's type.  float elements with
    # an int init have no precompiled kernel: the kernel templates take the call under hipcc, and a
    # host compiler is told so instead of silently accumulating in another type.
    body = """
        #include <thrust/device_vector.h>
        #include <thrust/scan.h>
        int main() { thrust::device_vector<float> d(10), o(10); thrust::exclusive_scan(d.begin(), d.end(), o.begin(), 0); }"""
    r = compile_snippet(tmp_path, body)
    assert r.returncode != 0
    assert "compile this translation unit with hipcc" in r.stderr
    src = tmp_path / "t.cpp"
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only",
                        "-I", INC, str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_another_device_system_is_refused(tmp_path):
    # thrust/detail/config/device_system.h:20-43: the system is chosen by -DTHRUST_DEVICE_SYSTEM
    body = """
        #include <thrust/device_vector.h>
        int main() { return THRUST_DEVICE_SYSTEM; }"""
    assert compile_snippet(tmp_path, body).returncode == 0
    assert compile_snippet(tmp_path, body, extra=("-DTHRUST_DEVICE_SYSTEM=THRUST_DEVICE_SYSTEM_CDNA4",)).returncode == 0
    r = compile_snippet(tmp_path, body, extra=("-DTHRUST_DEVICE_SYSTEM=THRUST_DEVICE_SYSTEM_OMP",))
    assert r.returncode != 0 and "cdna4 device system only" in r.stderr


def test_user_functor_on_device_range_needs_hipcc(tmp_path):
    body = """
        #include <thrust/device_vector.h>
        #include <thrust/transform.h>
        #include <thrust/reduce.h>
        struct twice { THRUST_CDNA4_HD int operator()(int x) const { return 2 * x; } };
        int main() { thrust::device_vector<int> d(10), o(10); thrust::transform(d.begin(), d.end(), o.begin(), twice());
                     return thrust::reduce(o.begin(), o.end(), 0); }"""
    r = compile_snippet(tmp_path, body)
    assert r.returncode != 0
    assert "compile this translation unit with hipcc" in r.stderr
    src = tmp_path / "t.cpp"
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only",
                        "-I", INC, str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_host_ranges_with_functors_build_with_gxx(tmp_path):
    r = compile_snippet(tmp_path, """
        #include <thrust/host_vector.h>
        #include <thrust/transform.h>
        #include <thrust/reduce.h>
        #include <thrust/sequence.h>
        #include <thrust/count.h>
        int main() { thrust::host_vector<int> h(10), o(10); thrust::sequence(h.begin(), h.end());
                     thrust::transform(h.begin(), h.end(), o.begin(), thrust::negate<int>());
                     return thrust::reduce(o.begin(), o.end()) + (int)thrust::count(o.begin(), o.end(), -3); }""")
    assert r.returncode == 0, r.stderr[-3000:]


def test_select_family_on_device_range_needs_hipcc(tmp_path):
    body = """
        #include <thrust/device_vector.h>
        #include <thrust/copy.h>
        #include <thrust/remove.h>
        #include <thrust/unique.h>
        struct odd { THRUST_CDNA4_HD bool operator()(int x) const { return x & 1; } };
        int main() { thrust::device_vector<int> d(10), o(10), v(10);
                     auto e = thrust::copy_if(d.begin(), d.end(), o.begin(), odd());
                     auto r = thrust::remove_if(d.begin(), d.end(), odd());
                     auto u = thrust::unique(d.begin(), d.end());
                     auto p = thrust::unique_by_key(d.begin(), d.end(), v.begin());
                     return (int)((e - o.begin()) + (r - d.begin()) + (u - d.begin()) + (p.first - d.begin())); }"""
    r = compile_snippet(tmp_path, body)
    assert r.returncode != 0
    assert "compile this translation unit with hipcc" in r.stderr
    src = tmp_path / "t.cpp"
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only",
                        "-I", INC, str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_select_family_on_host_ranges_builds_with_gxx(tmp_path):
    r = compile_snippet(tmp_path, """
        #include <thrust/host_vector.h>
        #include <thrust/copy.h>
        #include <thrust/remove.h>
        #include <thrust/unique.h>
        struct odd { bool operator()(int x) const { return x & 1; } };
        int main() { thrust::host_vector<int> h(10), o(10), v(10);
                     auto e = thrust::copy_if(h.begin(), h.end(), o.begin(), odd());
                     auto r = thrust::remove(h.begin(), h.end(), 3);
                     auto u = thrust::unique(h.begin(), h.end());
                     auto p = thrust::unique_by_key(h.begin(), h.end(), v.begin());
                     return (int)((e - o.begin()) + (r - h.begin()) + (u - h.begin()) + (p.first - h.begin())); }""")
    assert r.returncode == 0, r.stderr[-3000:]


def test_every_public_header_compiles_on_its_own(tmp_path):
    """Each header under include/thrust (not detail/) is self-contained under g++."""
    import glob
    headers = sorted(h for h in glob.glob(os.path.join(INC, "thrust", "**", "*.h"), recursive=True) if "/detail/" not in h)
    stubs = [h for h in headers if "is not provided by the cdna4 device system" in open(h).read()]
    for h in stubs:  # a header of the reference that is not provided stops the build with that message
        r = compile_snippet(tmp_path, '#include <%s>\nint main() { return 0; }\n' % os.path.relpath(h, INC))
        assert r.returncode != 0 and "is not provided by the cdna4 device system" in r.stderr, h
    headers = [h for h in headers if h not in stubs]
    assert len(headers) > 70
    body = "".join('#include <%s>\n' % os.path.relpath(h, INC) for h in headers) + "int main() { return 0; }\n"
    r = compile_snippet(tmp_path, body)
    assert r.returncode == 0, r.stderr[-3000:]
    for h in headers:  # and each one alone
        r = compile_snippet(tmp_path, '#include <%s>\nint main() { return 0; }\n' % os.path.relpath(h, INC))
        assert r.returncode == 0, (h, r.stderr[-2000:])


# the per-algorithm headers a device system's directory holds: one for every name under the
# reference's thrust/system/detail/adl/ (each adl/<name>.h includes <system root>/detail/<name>.h)
SYSTEM_DETAIL_NAMES = """adjacent_difference assign_value binary_search copy copy_if count equal extrema fill find for_each
gather generate get_value inner_product iter_swap logical malloc_and_free merge mismatch partition per_device_resource
reduce reduce_by_key remove replace reverse scan scan_by_key scatter sequence set_operations sort swap_ranges tabulate
temporary_buffer transform transform_reduce transform_scan uninitialized_copy uninitialized_fill unique unique_by_key""".split()


def test_the_system_directory_has_the_reference_layout(tmp_path):
    """thrust/system/cdna4/ holds what the reference asks of a device system's directory
    (thrust/system/cuda/: execution_policy.h, memory.h, memory_resource.h, pointer.h, vector.h,
    detail/execution_policy.h, detail/par.h and one detail/<algorithm>.h per name of
    thrust/system/detail/adl/), and each of these headers compiles when it is the first one included."""
    root = os.path.join(INC, "thrust", "system", "cdna4")
    assert len(SYSTEM_DETAIL_NAMES) == 43
    names = (["execution_policy.h", "memory.h", "memory_resource.h", "pointer.h", "vector.h", "detail/execution_policy.h", "detail/par.h"]
             + ["detail/%s.h" % n for n in SYSTEM_DETAIL_NAMES])
    for n in names:
        assert os.path.exists(os.path.join(root, n)), n
    ref = "/root/reference/thrust/system/detail/adl"
    if os.path.isdir(ref):  # the list above is the reference's
        assert sorted(f[:-2] for f in os.listdir(ref) if f.endswith(".h")) == sorted(SYSTEM_DETAIL_NAMES)
    for n in names:
        r = compile_snippet(tmp_path, '#include <thrust/system/cdna4/%s>\nint main() { return 0; }\n' % n)
        assert r.returncode == 0, (n, r.stderr[-2000:])
