// Throughput of the comparison sort (kernel templates instantiated with a user comparator):
// prints one JSON object.  Inputs are resident on the device when the timed region starts; the
// unsorted input is restored between repetitions outside of it.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <algorithm>
#include <cstdlib>
#include <functional>
#include <vector>

#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/sort.h>

struct my_less {
  __host__ __device__ bool operator()(unsigned a, unsigned b) const { return a < b; }
};

static std::uint64_t splitmix64(std::uint64_t& x) {
  std::uint64_t z = (x += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

template <class F>
static float median_ms(F run, F restore, int reps) {
  hipEvent_t a, b;
  hipEventCreate(&a);
  hipEventCreate(&b);
  std::vector<float> ms;
  for (int r = 0; r < reps + 1; r++) {
    restore();
    hipDeviceSynchronize();
    hipEventRecord(a, 0);
    run();
    hipEventRecord(b, 0);
    hipEventSynchronize(b);
    float t;
    hipEventElapsedTime(&t, a, b);
    if (r) ms.push_back(t);  // the first repetition warms the allocator pool
  }
  std::sort(ms.begin(), ms.end());
  return ms[ms.size() / 2];
}

int main(int argc, char** argv) {
  const int log2n = argc > 1 ? std::atoi(argv[1]) : 26;
  const std::size_t n = std::size_t(1) << log2n;
  std::vector<unsigned> h(n);
  std::uint64_t s = 1337;
  for (std::size_t i = 0; i < n; i++) h[i] = (unsigned)splitmix64(s);
  thrust::device_vector<unsigned> src(h), keys(n), vals(n);

  std::function<void()> restore = [&] { keys = src; };
  std::function<void()> run_keys = [&] { thrust::sort(thrust::cdna4::par_nosync, keys.begin(), keys.end(), my_less()); };
  const float ms_keys = median_ms(run_keys, restore, 5);
  std::vector<unsigned> out(n);
  hipMemcpy(out.data(), thrust::raw_pointer_cast(keys.data()), n * 4, hipMemcpyDeviceToHost);
  bool ok = true;
  for (std::size_t i = 1; i < n; i++) {
    if (out[i - 1] > out[i]) {
      if (ok) std::fprintf(stderr, "first inversion at %zu: %u > %u\n", i, out[i - 1], out[i]);
      ok = false;
    }
  }

  std::function<void()> run_pairs = [&] {
    thrust::sort_by_key(thrust::cdna4::par_nosync, keys.begin(), keys.end(), vals.begin(), my_less());
  };
  const float ms_pairs = median_ms(run_pairs, restore, 5);

  // passes over the data: one tile sort + ceil(log2(n / tile)) merges, each reading and writing every item
  namespace ms = thrust::system::cdna4::detail::merge;
  auto passes_of = [&](int items_per_thread) {
    int p = 1;
    for (std::size_t w = (std::size_t)ms::kBlock * items_per_thread; w < n; w *= 2) p++;
    return p;
  };
  const int passes = passes_of(ms::items_per_thread<unsigned, ms::no_value>());
  const int passes_pairs = passes_of(ms::items_per_thread<unsigned, unsigned>());
  std::printf(
      "{\"merge_sort_u32_custom_less\": {\"value\": %.3f, \"unit\": \"Gkeys/s\", \"ms\": %.3f, \"n\": %zu, \"passes\": %d, "
      "\"traffic_GBs\": %.1f, \"sorted\": %s}, \"merge_sort_by_key_u32_u32_custom_less\": {\"value\": %.3f, \"unit\": "
      "\"Gkeys/s\", \"ms\": %.3f, \"traffic_GBs\": %.1f}}\n",
      n / ms_keys / 1e6, ms_keys, n, passes, passes * 8.0 * n / ms_keys / 1e6, ok ? "true" : "false", n / ms_pairs / 1e6,
      ms_pairs, passes_pairs * 16.0 * n / ms_pairs / 1e6);
  return ok ? 0 : 1;
}
