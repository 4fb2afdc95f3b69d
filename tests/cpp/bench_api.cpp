// Throughput as a caller of the Thrust API sees it: wall-clock time around the synchronous calls
// thrust::sort(d.begin(), d.end()) and thrust::inclusive_scan(thrust::device, ...), so the header
// dispatch, the temporary-storage pool, the launches and the final synchronisation are all inside
// the timed region.  The first call of the process is reported on its own (it also pays for loading
// the code object, the pool's first allocation and the sort's once-per-device LDS check).  Also the
// user-operator scan / reduce_by_key engine on the same inputs as the precompiled kernels.
// One JSON object on the last line.  A plain host translation unit unless built by hipcc, which
// adds the user-operator cases.
#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <string>
#include <vector>

#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/host_vector.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sort.h>

using clk = std::chrono::steady_clock;
static double ms_since(clk::time_point t0) { return std::chrono::duration<double, std::milli>(clk::now() - t0).count(); }

static double median_ms(const std::function<void()>& prepare, const std::function<void()>& run, int reps) {
  std::vector<double> ms;
  for (int r = 0; r < reps + 1; r++) {
    prepare();
    thrust_cdna4_stream_synchronize(nullptr);
    const auto t0 = clk::now();
    run();  // synchronous: returns when the result is there
    const double t = ms_since(t0);
    if (r >= 1) ms.push_back(t);
  }
  std::sort(ms.begin(), ms.end());
  return ms[ms.size() / 2];
}

#if defined(__HIPCC__)
// a user operator the library has no precompiled kernel for: the kernel templates take the call
struct my_plus {
  __host__ __device__ int operator()(int a, int b) const { return a + b; }
};
struct my_equal {
  __host__ __device__ bool operator()(int a, int b) const { return a == b; }
};
#endif

int main(int argc, char** argv) {
  const int log2n = argc > 1 ? std::atoi(argv[1]) : 28;
  const std::size_t n = std::size_t(1) << log2n;
  std::string out = "{";
  char buf[512];

  // ---- the very first Thrust call of the process: a 2^20-key sort
  thrust::host_vector<std::uint32_t> h(n);
  std::uint64_t s = 1337;
  for (auto& x : h) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    x = (std::uint32_t)(s >> 32);
  }
  {
    const auto t0 = clk::now();
    thrust::device_vector<std::uint32_t> first(h.begin(), h.begin() + (1 << 20));
    const double t_alloc = ms_since(t0);
    const auto t1 = clk::now();
    thrust::sort(first.begin(), first.end());
    const double t_sort = ms_since(t1);
    const auto t2 = clk::now();
    thrust::sort(first.begin(), first.end());
    const double t_again = ms_since(t2);
    std::snprintf(buf, sizeof buf,
                  "\"api_cold_start_ms\": {\"first_device_vector_2^20_u32\": %.2f, \"first_sort_2^20_u32\": %.3f, "
                  "\"second_sort_2^20_u32\": %.3f}, ",
                  t_alloc, t_sort, t_again);
    out += buf;
  }

  thrust::device_vector<std::uint32_t> src = h, d(n);
  // ---- thrust::sort, keys restored from a device copy outside the timed call
  out += "\"api_sort_u32_gkeys_per_s\": {";
  for (int lg : {20, 24, log2n}) {
    const std::size_t m = std::size_t(1) << lg;
    if (m > n) continue;
    const double ms = median_ms([&] { thrust::copy(src.begin(), src.begin() + m, d.begin()); },
                                [&] { thrust::sort(d.begin(), d.begin() + m); }, 10);
    std::snprintf(buf, sizeof buf, "\"2^%d\": %.3f, ", lg, m / ms / 1e6);
    out += buf;
  }
  out.resize(out.size() - 2);
  out += "}, ";
  {  // the first large sort above paid for the pool's growth; a cold large call on its own:
    thrust_cdna4_pool_trim();
    thrust::copy(src.begin(), src.end(), d.begin());
    thrust_cdna4_stream_synchronize(nullptr);
    const auto t0 = clk::now();
    thrust::sort(d.begin(), d.end());
    std::snprintf(buf, sizeof buf, "\"api_sort_u32_2^%d_with_an_empty_pool_ms\": %.3f, ", log2n, ms_since(t0));
    out += buf;
    if (!thrust::is_sorted(d.begin(), d.end())) {
      std::fprintf(stderr, "bench_api: sort result is not sorted\n");
      return 1;
    }
  }

  // ---- thrust::inclusive_scan(thrust::device, ...) over the size sweep
  thrust::device_vector<int> x(n, 1), y(n);
  out += "\"api_inclusive_scan_i32_gelem_per_s\": {";
  for (int lg = 20; lg <= log2n; lg += 2) {
    const std::size_t m = std::size_t(1) << lg;
    const double ms = median_ms([] {}, [&] { thrust::inclusive_scan(thrust::device, x.begin(), x.begin() + m, y.begin()); }, 10);
    std::snprintf(buf, sizeof buf, "\"2^%d\": %.2f, ", lg, m / ms / 1e6);
    out += buf;
  }
  out.resize(out.size() - 2);
  out += "}";
  if ((std::size_t)y[n - 1] != n) {
    std::fprintf(stderr, "bench_api: scan result is wrong\n");
    return 1;
  }

#if defined(__HIPCC__)
  // ---- the same scan and a reduce_by_key through the user-operator engine (kernel templates)
  {
    const double ms_b = median_ms([] {}, [&] { thrust::inclusive_scan(thrust::device, x.begin(), x.end(), y.begin()); }, 10);
    const double ms_g = median_ms([] {}, [&] { thrust::inclusive_scan(thrust::device, x.begin(), x.end(), y.begin(), my_plus()); }, 10);
    if ((std::size_t)y[n - 1] != n) {
      std::fprintf(stderr, "bench_api: user-operator scan result is wrong\n");
      return 1;
    }
    // keys: runs of 8
    thrust::device_vector<int> keys(n), ko(n), vo(n);
    {
      thrust::host_vector<int> hk(n);
      for (std::size_t i = 0; i < n; i++) hk[i] = (int)(i >> 3);
      keys = hk;
    }
    const double ms_rb = median_ms([] {}, [&] { thrust::reduce_by_key(thrust::device, keys.begin(), keys.end(), x.begin(), ko.begin(), vo.begin()); }, 10);
    const double ms_rg = median_ms([] {}, [&] {
      thrust::reduce_by_key(thrust::device, keys.begin(), keys.end(), x.begin(), ko.begin(), vo.begin(), my_equal(), my_plus());
    }, 10);
    if (vo[0] != 8 || vo[n / 8 - 1] != 8) {
      std::fprintf(stderr, "bench_api: user-operator reduce_by_key result is wrong\n");
      return 1;
    }
    std::snprintf(buf, sizeof buf,
                  ", \"api_user_operator_engine_2^%d_i32\": {\"inclusive_scan_builtin_plus_gelem_per_s\": %.2f, "
                  "\"inclusive_scan_user_plus_gelem_per_s\": %.2f, \"reduce_by_key_runs_of_8_builtin_gelem_per_s\": %.2f, "
                  "\"reduce_by_key_runs_of_8_user_ops_gelem_per_s\": %.2f}",
                  log2n, n / ms_b / 1e6, n / ms_g / 1e6, n / ms_rb / 1e6, n / ms_rg / 1e6);
    out += buf;
  }
#endif
  out += "}";
  std::printf("%s\n", out.c_str());
  return 0;
}
