// System-level behaviour of the cdna4 device system: execution policies and streams
// (testing/cuda/sort.cu:108-133, testing/cuda/scan.cu:123-215), par_nosync
// (testing/cuda/reduce_by_key.cu:202-206), allocation failure without terminate
// (testing/out_of_memory_recovery.cu:23-33), pointer reuse by the cached allocator
// (testing/caching_allocator.cu:6-17), empty ranges, containers, histogram extension.
#include <hip/hip_runtime_api.h>

#include <thrust/copy.h>
#include <thrust/fill.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sort.h>
#include <thrust/system/cdna4/histogram.h>
#include <thrust/system_error.h>

#include "testing.h"

void TestSortOnStream() {
  hipStream_t s;
  ASSERT_EQUAL((int)hipStreamCreate(&s), 0);
  thrust::host_vector<int> h = unittest::random_integers<int>(100003);
  thrust::device_vector<int> d = h;
  thrust::sort(thrust::cdna4::par.on(s), d.begin(), d.end());
  std::sort(h.begin(), h.end());
  ASSERT_EQUAL(h, d);
  // par_nosync returns without waiting: synchronise the stream before looking
  thrust::device_vector<int> d2 = unittest::random_integers<int>(100003);
  thrust::host_vector<int> h2 = d2;
  thrust::device_vector<int> out(d2.size());
  thrust::inclusive_scan(thrust::cdna4::par_nosync.on(s), d2.begin(), d2.end(), out.begin());
  ASSERT_EQUAL((int)hipStreamSynchronize(s), 0);
  thrust::host_vector<int> ho(h2.size());
  thrust::inclusive_scan(h2.begin(), h2.end(), ho.begin());
  ASSERT_EQUAL(ho, out);
  // reduce_by_key reads its run count back, so it is complete on return even under par_nosync
  thrust::device_vector<int> keys(1000, 7), vals(1000, 2), ko(1000), vo(1000);
  auto e = thrust::reduce_by_key(thrust::cdna4::par_nosync.on(s), keys.begin(), keys.end(), vals.begin(), ko.begin(),
                                 vo.begin());
  ASSERT_EQUAL(e.first - ko.begin(), 1);
  ASSERT_EQUAL((int)vo[0], 2000);
  ASSERT_EQUAL((int)hipStreamDestroy(s), 0);
}
DECLARE_UNITTEST(TestSortOnStream);

// fill / fill_n / copy / copy_n with execution policies (testing/fill.cu:20-110, copy.cu:100-180,
// copy_n.cu): contiguous ranges of arithmetic types need no device compiler in the caller
void TestFillAndCopyWithPolicies() {
  hipStream_t s;
  ASSERT_EQUAL((int)hipStreamCreate(&s), 0);
  thrust::device_vector<int> v(5, 0);
  thrust::fill(thrust::device, v.begin() + 1, v.begin() + 4, 7);
  ASSERT_EQUAL(v, thrust::host_vector<int>({0, 7, 7, 7, 0}));
  auto e = thrust::fill_n(v.begin(), 3, 2);
  ASSERT_EQUAL(e - v.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(v, thrust::host_vector<int>({2, 2, 2, 7, 0}));
  thrust::device_vector<double> big(100003), copy(100003);
  thrust::fill(thrust::cdna4::par.on(s), big.begin(), big.end(), 1.5);
  auto ce = thrust::copy(thrust::cdna4::par.on(s), big.begin(), big.end(), copy.begin());
  ASSERT_TRUE(ce == copy.end());
  ASSERT_EQUAL(copy, thrust::host_vector<double>(100003, 1.5));
  thrust::device_vector<double> head(10);
  thrust::copy_n(thrust::device, big.begin(), 10, head.begin());
  ASSERT_EQUAL(head, thrust::host_vector<double>(10, 1.5));
  thrust::host_vector<short> h(9);
  thrust::fill(thrust::host, h.begin(), h.end(), (short)-3);
  thrust::device_vector<short> d(9);
  thrust::copy_n(h.begin(), 9, d.begin());
  ASSERT_EQUAL(d, h);
  ASSERT_EQUAL((int)hipStreamDestroy(s), 0);
}
DECLARE_UNITTEST(TestFillAndCopyWithPolicies);

// thrust/device_vector.h: erase / insert / pop_back / shrink_to_fit (testing/vector_manipulation.cu,
// vector_insert.cu); erase(new_end, end()) is how remove_if / unique results are trimmed
void TestDeviceVectorEraseInsert() {
  thrust::device_vector<int> v(thrust::host_vector<int>({0, 1, 2, 3, 4, 5, 6, 7}));
  auto it = v.erase(v.begin() + 2, v.begin() + 5);
  ASSERT_EQUAL(it - v.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(v, thrust::host_vector<int>({0, 1, 5, 6, 7}));
  v.erase(v.begin());
  ASSERT_EQUAL(v, thrust::host_vector<int>({1, 5, 6, 7}));
  v.erase(v.begin() + 2, v.end());
  ASSERT_EQUAL(v, thrust::host_vector<int>({1, 5}));
  const int more[3] = {8, 9, 10};
  v.insert(v.begin() + 1, more, more + 3);
  ASSERT_EQUAL(v, thrust::host_vector<int>({1, 8, 9, 10, 5}));
  thrust::device_vector<int> d2(2, 4);
  v.insert(v.end(), d2.begin(), d2.end());
  v.insert(v.begin(), -1);
  ASSERT_EQUAL(v, thrust::host_vector<int>({-1, 1, 8, 9, 10, 5, 4, 4}));
  v.pop_back();
  v.shrink_to_fit();
  ASSERT_EQUAL(v.size(), (std::size_t)7);
  ASSERT_EQUAL(v.capacity(), (std::size_t)7);
  ASSERT_EQUAL((int)v.back(), 4);
}
DECLARE_UNITTEST(TestDeviceVectorEraseInsert);

void TestEmptyRanges() {
  thrust::device_vector<int> d, o;
  thrust::sort(d.begin(), d.end());
  thrust::sort_by_key(d.begin(), d.end(), o.begin());
  ASSERT_TRUE(thrust::inclusive_scan(d.begin(), d.end(), o.begin()) == o.begin());
  ASSERT_TRUE(thrust::exclusive_scan(d.begin(), d.end(), o.begin(), 5) == o.begin());
  auto e = thrust::reduce_by_key(d.begin(), d.end(), d.begin(), o.begin(), o.begin());
  ASSERT_TRUE(e.first == o.begin() && e.second == o.begin());
}
DECLARE_UNITTEST(TestEmptyRanges);

void TestOutOfMemoryRecovery() {
  // an absurd request throws bad_alloc and leaves the system usable
  ASSERT_THROWS(thrust::device_vector<char> big((std::size_t)1 << 50), std::bad_alloc);
  thrust::device_vector<int> d(4, 3);
  ASSERT_EQUAL((int)d[2], 3);
  // a failing C-ABI call surfaces as thrust::system_error with the cdna4 category
  try {
    thrust::system::cdna4::detail::throw_on_error(1, "probe");
    ASSERT_TRUE(false);
  } catch (const thrust::system_error& e) {
    ASSERT_TRUE(e.code().category() == thrust::cdna4_category());
    ASSERT_EQUAL(e.code().value(), 1);
  }
}
DECLARE_UNITTEST(TestOutOfMemoryRecovery);

void TestCachedAllocatorReusesBlocks() {
  void* a = nullptr;
  void* b = nullptr;
  ASSERT_EQUAL(thrust_cdna4_malloc(&a, 1000, nullptr), 0);
  ASSERT_EQUAL(thrust_cdna4_free(a, nullptr), 0);
  ASSERT_EQUAL(thrust_cdna4_malloc(&b, 900, nullptr), 0);  // same size class, same stream: no driver call
  ASSERT_TRUE(a == b);
  ASSERT_EQUAL(thrust_cdna4_free(b, nullptr), 0);
  const std::size_t held = thrust_cdna4_pool_bytes();
  ASSERT_TRUE(held >= 1024);
  ASSERT_EQUAL(thrust_cdna4_free(b, nullptr) != 0, true);  // double free is reported, not fatal
  ASSERT_EQUAL(thrust_cdna4_pool_trim(), 0);
  ASSERT_TRUE(thrust_cdna4_pool_bytes() < held);
}
DECLARE_UNITTEST(TestCachedAllocatorReusesBlocks);

void TestDeviceVectorBasics() {
  thrust::device_vector<float> d(5);
  ASSERT_EQUAL((float)d[3], 0.0f);
  d[3] = 2.5f;
  ASSERT_EQUAL((float)d[3], 2.5f);
  thrust::fill(d.begin(), d.begin() + 2, 7);
  thrust::host_vector<float> h = d;
  ASSERT_EQUAL(h[0], 7.0f);
  ASSERT_EQUAL(h[1], 7.0f);
  ASSERT_EQUAL(h[2], 0.0f);
  d.resize(9, 1.0f);
  ASSERT_EQUAL(d.size(), std::size_t(9));
  ASSERT_EQUAL((float)d[8], 1.0f);
  ASSERT_EQUAL((float)d[3], 2.5f);
  thrust::device_vector<float> c = d;
  ASSERT_EQUAL(c, d);
  d.push_back(4.0f);
  ASSERT_EQUAL((float)d.back(), 4.0f);
  thrust::host_vector<float> back(d.size());
  thrust::copy(d.begin(), d.end(), back.begin());
  ASSERT_EQUAL(back, d);
  thrust::device_vector<float> e(d.size());
  thrust::copy(back.begin(), back.end(), e.begin());
  ASSERT_EQUAL(e, d);
  thrust::device_ptr<float> p = thrust::device_malloc<float>(16);
  thrust::fill(p, p + 16, 3.0f);
  ASSERT_EQUAL((float)p[15], 3.0f);
  thrust::device_free(p);
}
DECLARE_UNITTEST(TestDeviceVectorBasics);

// internal/test/thrust.example.histogram.filecheck:1-5
void TestHistogramExample() {
  const int data[40] = {3, 4, 3, 5, 8, 5, 6, 6, 4, 4, 5, 3, 2, 5, 6, 3, 1, 3, 2, 3,
                        6, 5, 3, 3, 3, 2, 4, 2, 3, 3, 2, 5, 5, 5, 8, 2, 5, 6, 6, 3};
  const unsigned expected[9] = {0, 1, 6, 12, 4, 9, 6, 0, 2};
  thrust::device_vector<int> d(data, data + 40);
  thrust::device_vector<unsigned> counts(9);
  thrust::cdna4::histogram_even(d.begin(), d.end(), counts.begin(), 9, 0.0, 9.0);
  ASSERT_EQUAL(counts, thrust::host_vector<unsigned>(expected, expected + 9));
}
DECLARE_UNITTEST(TestHistogramExample);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
