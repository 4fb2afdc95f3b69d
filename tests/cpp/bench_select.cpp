// Throughput of the stable-compaction algorithms (kernel templates instantiated with user
// predicates): copy_if keeping half of 2^28 random ints, unique_copy over runs of mean length 4,
// unique_by_key_copy with 4-byte values; one JSON object.  Algorithmic bytes = one read of the
// input plus one write of what is kept.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <vector>

#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/sequence.h>
#include <thrust/transform.h>
#include <thrust/unique.h>

struct hash_of {
  __host__ __device__ int operator()(int i) const {
    unsigned x = (unsigned)i * 2654435761u;
    x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
    return (int)x;
  }
};
struct run_of {  // runs of 4 equal values
  __host__ __device__ int operator()(int i) const { return hash_of()(i >> 2); }
};
struct is_even {
  __host__ __device__ bool operator()(int x) const { return (x & 1) == 0; }
};

static float median_ms(const std::function<void()>& run, int reps) {
  hipEvent_t a, b;
  hipEventCreate(&a);
  hipEventCreate(&b);
  std::vector<float> ms;
  for (int r = 0; r < reps + 2; r++) {
    hipDeviceSynchronize();
    hipEventRecord(a, 0);
    run();
    hipEventRecord(b, 0);
    hipEventSynchronize(b);
    float t;
    hipEventElapsedTime(&t, a, b);
    if (r >= 2) ms.push_back(t);
  }
  std::sort(ms.begin(), ms.end());
  return ms[ms.size() / 2];
}

int main(int argc, char** argv) {
  const int log2n = argc > 1 ? std::atoi(argv[1]) : 28;
  const std::size_t n = std::size_t(1) << log2n;
  thrust::device_vector<int> idx(n), x(n), v(n), out(n), vout(n);
  thrust::sequence(idx.begin(), idx.end());
  thrust::transform(idx.begin(), idx.end(), x.begin(), hash_of());
  std::ptrdiff_t kept = 0, heads = 0, heads2 = 0;
  const float ms_c = median_ms([&] { kept = thrust::copy_if(x.begin(), x.end(), out.begin(), is_even()) - out.begin(); }, 10);
  thrust::transform(idx.begin(), idx.end(), x.begin(), run_of());
  const float ms_u = median_ms([&] { heads = thrust::unique_copy(x.begin(), x.end(), out.begin()) - out.begin(); }, 10);
  const float ms_k = median_ms([&] {
    heads2 = thrust::unique_by_key_copy(x.begin(), x.end(), idx.begin(), out.begin(), vout.begin()).first - out.begin(); }, 10);
  const double bc = 4.0 * n + 4.0 * kept, bu = 4.0 * n + 4.0 * heads, bk = 8.0 * n + 8.0 * heads2;
  std::printf(
      "{\"copy_if_i32_half\": {\"value\": %.1f, \"unit\": \"Gelem/s\", \"ms\": %.4f, \"kept\": %td, \"algorithmic_bytes\": %.0f, \"roofline_frac\": %.4f}, "
      "\"unique_copy_i32_runs4\": {\"value\": %.1f, \"unit\": \"Gelem/s\", \"ms\": %.4f, \"kept\": %td, \"algorithmic_bytes\": %.0f, \"roofline_frac\": %.4f}, "
      "\"unique_by_key_copy_i32_i32_runs4\": {\"value\": %.1f, \"unit\": \"Gelem/s\", \"ms\": %.4f, \"kept\": %td, \"algorithmic_bytes\": %.0f, \"roofline_frac\": %.4f}}\n",
      n / ms_c / 1e6, ms_c, kept, bc, bc / ms_c / 1e6 / 8000.0, n / ms_u / 1e6, ms_u, heads, bu, bu / ms_u / 1e6 / 8000.0,
      n / ms_k / 1e6, ms_k, heads2, bk, bk / ms_k / 1e6 / 8000.0);
  return 0;
}
