// Throughput of the generic-functor algorithms (kernel templates instantiated with user
// functors): transform (saxpy), reduce and transform_reduce at 2^28 elements; one JSON object.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <vector>

#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/reduce.h>
#include <thrust/sequence.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>

struct saxpy {
  float a;
  __host__ __device__ float operator()(float x, float y) const { return a * x + y; }
};
struct square {
  __host__ __device__ float operator()(float x) const { return x * x; }
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
  thrust::device_vector<float> x(n), y(n), z(n);
  thrust::sequence(x.begin(), x.end(), 0.0f, 1e-6f);
  thrust::sequence(y.begin(), y.end(), 1.0f, 0.0f);
  volatile float sink = 0;
  const float ms_t = median_ms([&] { thrust::transform(thrust::cdna4::par_nosync, x.begin(), x.end(), y.begin(), z.begin(), saxpy{2.0f}); }, 10);
  const float ms_r = median_ms([&] { sink = thrust::reduce(x.begin(), x.end(), 0.0f); }, 10);
  const float ms_tr = median_ms([&] { sink = thrust::transform_reduce(x.begin(), x.end(), square(), 0.0f, thrust::plus<float>()); }, 10);
  (void)sink;
  std::printf(
      "{\"transform_saxpy_f32\": {\"value\": %.1f, \"unit\": \"Gelem/s\", \"ms\": %.4f, \"algorithmic_bytes\": %.0f, \"roofline_frac\": %.4f}, "
      "\"reduce_f32\": {\"value\": %.1f, \"unit\": \"Gelem/s\", \"ms\": %.4f, \"algorithmic_bytes\": %.0f, \"roofline_frac\": %.4f}, "
      "\"transform_reduce_f32\": {\"value\": %.1f, \"unit\": \"Gelem/s\", \"ms\": %.4f, \"algorithmic_bytes\": %.0f, \"roofline_frac\": %.4f}}\n",
      n / ms_t / 1e6, ms_t, 12.0 * n, 12.0 * n / ms_t / 1e6 / 8000.0, n / ms_r / 1e6, ms_r, 4.0 * n, 4.0 * n / ms_r / 1e6 / 8000.0,
      n / ms_tr / 1e6, ms_tr, 4.0 * n, 4.0 * n / ms_tr / 1e6 / 8000.0);
  return 0;
}
