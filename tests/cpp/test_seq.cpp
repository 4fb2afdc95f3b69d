// thrust::seq: the sequential algorithms of the hot path, called on the host and from inside a
// kernel on ranges that belong to one thread (after the reference's testing/cuda/sort.cu:18-105,
// whose kernels call thrust::sort(thrust::seq, ...), and testing/scan.cu / reduce_by_key.cu for
// the expected values).  Compiled by hipcc: the second half launches kernels; `test_seq Host`
// runs the host half only.
#include <algorithm>
#include <numeric>
#include <random>
#include <vector>

#include <hip/hip_runtime.h>

#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sort.h>

#include "testing.h"

template <class T>
struct my_less {
  __host__ __device__ bool operator()(const T& a, const T& b) const { return a < b; }
};
struct by_tens {  // many equal keys: stability shows
  __host__ __device__ bool operator()(int a, int b) const { return a / 10 < b / 10; }
};

template <class T>
static std::vector<T> random_values(std::size_t n, unsigned seed, int lo, int hi) {
  std::mt19937 g(seed);
  std::uniform_int_distribution<int> d(lo, hi);
  std::vector<T> v(n);
  for (auto& x : v) x = (T)d(g);
  return v;
}

// ---------------------------------------------------------------- host
void TestSeqSortHost() {
  for (std::size_t n : {0u, 1u, 2u, 3u, 15u, 16u, 17u, 33u, 100u, 1000u, 4099u}) {
    std::vector<int> k = random_values<int>(n, 7 + (unsigned)n, -50, 50), ek = k;
    std::stable_sort(ek.begin(), ek.end());
    thrust::sort(thrust::seq, k.begin(), k.end());
    ASSERT_TRUE(k == ek);
    // stability: equal keys (by tens) keep their input order, values travel with their keys
    std::vector<int> keys = random_values<int>(n, 11 + (unsigned)n, 0, 99), vals(n);
    std::iota(vals.begin(), vals.end(), 0);
    std::vector<int> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return keys[a] / 10 < keys[b] / 10; });
    std::vector<int> want_k(n), want_v(n);
    for (std::size_t i = 0; i < n; i++) { want_k[i] = keys[order[i]]; want_v[i] = order[i]; }
    thrust::stable_sort_by_key(thrust::seq, keys.begin(), keys.end(), vals.begin(), by_tens());
    ASSERT_TRUE(keys == want_k);
    ASSERT_TRUE(vals == want_v);
    std::vector<int> desc = random_values<int>(n, 13 + (unsigned)n, -9, 9), ed = desc;
    std::stable_sort(ed.begin(), ed.end(), std::greater<int>());
    thrust::stable_sort(thrust::seq, desc.begin(), desc.end(), thrust::greater<int>());
    ASSERT_TRUE(desc == ed);
  }
}

void TestSeqScansAndReduceByKeyHost() {
  // testing/scan.cu TestScanSimple: {1,3,-2,4,-5}
  std::vector<int> in{1, 3, -2, 4, -5}, out(5);
  thrust::inclusive_scan(thrust::seq, in.begin(), in.end(), out.begin());
  ASSERT_TRUE((out == std::vector<int>{1, 4, 2, 6, 1}));
  thrust::exclusive_scan(thrust::seq, in.begin(), in.end(), out.begin());
  ASSERT_TRUE((out == std::vector<int>{0, 1, 4, 2, 6}));
  thrust::exclusive_scan(thrust::seq, in.begin(), in.end(), out.begin(), 3);
  ASSERT_TRUE((out == std::vector<int>{3, 4, 7, 5, 9}));
  thrust::inclusive_scan(thrust::seq, in.begin(), in.end(), out.begin(), thrust::maximum<int>());
  ASSERT_TRUE((out == std::vector<int>{1, 3, 3, 4, 4}));
  std::vector<int> inplace = in;
  thrust::exclusive_scan(thrust::seq, inplace.begin(), inplace.end(), inplace.begin(), 3);
  ASSERT_TRUE((inplace == std::vector<int>{3, 4, 7, 5, 9}));
  // testing/scan_by_key.cu TestInclusiveScanByKeySimple / TestExclusiveScanByKeySimple
  std::vector<int> keys{0, 1, 1, 1, 2, 3, 3}, vals{1, 2, 3, 4, 5, 6, 7}, o(7);
  thrust::inclusive_scan_by_key(thrust::seq, keys.begin(), keys.end(), vals.begin(), o.begin());
  ASSERT_TRUE((o == std::vector<int>{1, 2, 5, 9, 5, 6, 13}));
  thrust::exclusive_scan_by_key(thrust::seq, keys.begin(), keys.end(), vals.begin(), o.begin());
  ASSERT_TRUE((o == std::vector<int>{0, 0, 2, 5, 0, 0, 6}));
  thrust::exclusive_scan_by_key(thrust::seq, keys.begin(), keys.end(), vals.begin(), o.begin(), 10);
  ASSERT_TRUE((o == std::vector<int>{10, 10, 12, 15, 10, 10, 16}));
  // testing/reduce_by_key.cu TestReduceByKeySimple: keys 11 11 21 20 21 21 21 37 37, values 0..8
  std::vector<int> rk{11, 11, 21, 20, 21, 21, 21, 37, 37}, rv{0, 1, 2, 3, 4, 5, 6, 7, 8}, ko(9), vo(9);
  auto ends = thrust::reduce_by_key(thrust::seq, rk.begin(), rk.end(), rv.begin(), ko.begin(), vo.begin());
  ASSERT_TRUE(ends.first - ko.begin() == 5 && ends.second - vo.begin() == 5);
  ko.resize(5);
  vo.resize(5);
  ASSERT_TRUE((ko == std::vector<int>{11, 21, 20, 21, 37}));
  ASSERT_TRUE((vo == std::vector<int>{1, 2, 3, 15, 15}));
}

// ---------------------------------------------------------------- inside a kernel
template <class Policy, class It, class Compare>
__global__ void sort_kernel(Policy exec, It first, It last, Compare comp) {
  thrust::sort(exec, first, last, comp);
}
template <class Policy, class It>
__global__ void sort_kernel_default(Policy exec, It first, It last) {
  thrust::sort(exec, first, last);
}

template <class T, class Compare>
static void check_device_side_sort(std::size_t n, Compare comp) {
  thrust::host_vector<T> h(n);
  std::vector<T> r = random_values<T>(n, 3 + (unsigned)n, -100, 100);
  for (std::size_t i = 0; i < n; i++) h[i] = r[i];
  thrust::device_vector<T> d = h;
  hipLaunchKernelGGL((sort_kernel<decltype(thrust::seq), typename thrust::device_vector<T>::iterator, Compare>), dim3(1), dim3(1), 0, 0,
                     thrust::seq, d.begin(), d.end(), comp);
  ASSERT_TRUE(hipDeviceSynchronize() == hipSuccess);
  std::stable_sort(r.begin(), r.end(), comp);
  thrust::host_vector<T> got = d;
  bool same = true;
  for (std::size_t i = 0; i < n; i++) same = same && got[i] == r[i];
  ASSERT_TRUE(same);
}

// every thread sorts, scans and reduces a segment of its own
__global__ void per_thread_kernel(int* keys, int* vals, int* scanned, int* run_keys, int* run_sums, int* run_counts, int seg, int nseg) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nseg) return;
  int* k = keys + (size_t)t * seg;
  int* v = vals + (size_t)t * seg;
  thrust::sort_by_key(thrust::seq, k, k + seg, v);
  thrust::inclusive_scan(thrust::seq, v, v + seg, scanned + (size_t)t * seg);
  thrust::pair<int*, int*> ends = thrust::reduce_by_key(thrust::seq, k, k + seg, v, run_keys + (size_t)t * seg, run_sums + (size_t)t * seg);
  run_counts[t] = (int)(ends.first - (run_keys + (size_t)t * seg));
}

void TestSeqInsideKernels() {
  for (std::size_t n : {0u, 1u, 2u, 17u, 100u, 1000u}) {
    check_device_side_sort<int>(n, my_less<int>());
    check_device_side_sort<signed char>(n, my_less<signed char>());
    check_device_side_sort<int>(n, thrust::less<int>());
    check_device_side_sort<int>(n, thrust::greater<int>());
  }
  {  // without a comparator
    std::vector<int> r = random_values<int>(500, 99, -1000, 1000);
    thrust::device_vector<int> d(r.begin(), r.end());
    hipLaunchKernelGGL((sort_kernel_default<decltype(thrust::seq), int*>), dim3(1), dim3(1), 0, 0, thrust::seq,
                       thrust::raw_pointer_cast(d.data()), thrust::raw_pointer_cast(d.data()) + 500);
    ASSERT_TRUE(hipDeviceSynchronize() == hipSuccess);
    std::sort(r.begin(), r.end());
    thrust::host_vector<int> got = d;
    ASSERT_TRUE(std::equal(r.begin(), r.end(), got.begin()));
  }
  const int seg = 37, nseg = 300;
  std::vector<int> hk = random_values<int>((size_t)seg * nseg, 5, 0, 9), hv = random_values<int>((size_t)seg * nseg, 6, -5, 5);
  thrust::device_vector<int> dk(hk.begin(), hk.end()), dv(hv.begin(), hv.end()), ds((size_t)seg * nseg), drk((size_t)seg * nseg),
      drs((size_t)seg * nseg), drc(nseg);
  hipLaunchKernelGGL(per_thread_kernel, dim3((nseg + 63) / 64), dim3(64), 0, 0, thrust::raw_pointer_cast(dk.data()),
                     thrust::raw_pointer_cast(dv.data()), thrust::raw_pointer_cast(ds.data()), thrust::raw_pointer_cast(drk.data()),
                     thrust::raw_pointer_cast(drs.data()), thrust::raw_pointer_cast(drc.data()), seg, nseg);
  ASSERT_TRUE(hipDeviceSynchronize() == hipSuccess);
  thrust::host_vector<int> gk = dk, gv = dv, gs = ds, grk = drk, grs = drs, grc = drc;
  bool ok = true;
  for (int t = 0; t < nseg && ok; t++) {
    std::vector<int> order(seg);
    std::iota(order.begin(), order.end(), 0);
    const int* k0 = hk.data() + (size_t)t * seg;
    const int* v0 = hv.data() + (size_t)t * seg;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return k0[a] < k0[b]; });
    int sum = 0, runs = 0;
    for (int i = 0; i < seg; i++) {
      const int key = k0[order[i]], val = v0[order[i]];
      ok = ok && gk[(size_t)t * seg + i] == key && gv[(size_t)t * seg + i] == val;
      sum += val;
      ok = ok && gs[(size_t)t * seg + i] == sum;
      if (i == 0 || key != k0[order[i - 1]]) runs++;
    }
    ok = ok && grc[t] == runs;
    int r = -1, acc = 0;
    for (int i = 0; i < seg; i++) {
      const int key = k0[order[i]], val = v0[order[i]];
      if (i == 0 || key != k0[order[i - 1]]) {
        if (r >= 0) ok = ok && grs[(size_t)t * seg + r] == acc;
        r++;
        acc = 0;
        ok = ok && grk[(size_t)t * seg + r] == key;
      }
      acc += val;
    }
    ok = ok && grs[(size_t)t * seg + r] == acc;
  }
  ASSERT_TRUE(ok);
}

DECLARE_UNITTEST(TestSeqSortHost);
DECLARE_UNITTEST(TestSeqScansAndReduceByKeyHost);
DECLARE_UNITTEST(TestSeqInsideKernels);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
