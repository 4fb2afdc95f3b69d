// Sort tests in the shape of the reference's testing/sort.cu, sort_by_key.cu,
// stable_sort_by_key.cu, sort_variable_bits.cu: known answers plus host-vs-device
// comparison over the size ladder.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>

#include <thrust/version.h>
#include <thrust/functional.h>
#include <thrust/sort.h>

#include "testing.h"

static_assert(THRUST_CDNA4_VERSION >= 100, "<thrust/...> did not resolve to the cdna4 headers");

// testing/sort.cu:42-75
template <class T>
void TestSortSimple() {
  const T unsorted[7] = {1, 3, 6, 5, 2, 0, 4};
  thrust::device_vector<T> d(unsorted, unsorted + 7);
  thrust::host_vector<T> h(unsorted, unsorted + 7);
  thrust::host_vector<T> expected(7);
  for (int i = 0; i < 7; i++) expected[i] = (T)i;
  thrust::sort(d.begin(), d.end());
  thrust::sort(h.begin(), h.end());
  ASSERT_EQUAL(d, expected);
  ASSERT_EQUAL(h, expected);
}
DECLARE_TYPED_UNITTEST(TestSortSimple, int);
DECLARE_TYPED_UNITTEST(TestSortSimple, short);
DECLARE_TYPED_UNITTEST(TestSortSimple, char);
DECLARE_TYPED_UNITTEST(TestSortSimple, uint64_t);
DECLARE_TYPED_UNITTEST(TestSortSimple, float);
DECLARE_TYPED_UNITTEST(TestSortSimple, double);

// testing/sort.cu:79-104
template <class T>
void TestSortAscendingAndDescendingKey() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    thrust::device_vector<T> d = h;
    thrust::sort(h.begin(), h.end(), thrust::less<T>());
    thrust::sort(d.begin(), d.end(), thrust::less<T>());
    ASSERT_EQUAL(h, d);
    h = unittest::random_integers<T>(n, 99);
    d = h;
    thrust::sort(h.begin(), h.end(), thrust::greater<T>());
    thrust::sort(d.begin(), d.end(), thrust::greater<T>());
    ASSERT_EQUAL(h, d);
  }
}
DECLARE_TYPED_UNITTEST(TestSortAscendingAndDescendingKey, int);
DECLARE_TYPED_UNITTEST(TestSortAscendingAndDescendingKey, uint32_t);
DECLARE_TYPED_UNITTEST(TestSortAscendingAndDescendingKey, int8_t);
DECLARE_TYPED_UNITTEST(TestSortAscendingAndDescendingKey, uint16_t);
DECLARE_TYPED_UNITTEST(TestSortAscendingAndDescendingKey, int64_t);

void TestSortFloatKeys() {
  for (std::size_t n : {std::size_t(100), std::size_t(4099), std::size_t(300001)}) {
    thrust::host_vector<float> h = unittest::random_samples<float>(n);
    thrust::device_vector<float> d = h;
    thrust::sort(h.begin(), h.end());
    thrust::sort(d.begin(), d.end());
    ASSERT_EQUAL(h, d);
    thrust::host_vector<double> h2 = unittest::random_samples<double>(n);
    thrust::device_vector<double> d2 = h2;
    thrust::sort(h2.begin(), h2.end(), thrust::greater<double>());
    thrust::sort(d2.begin(), d2.end(), thrust::greater<double>());
    ASSERT_EQUAL(h2, d2);
  }
  // the bit-pattern total order of the reference's host radix sort: -0 before +0, denormals kept
  const float tiny = std::numeric_limits<float>::denorm_min();
  const float ordered[8] = {-INFINITY, -1.5f, -tiny, -0.0f, 0.0f, tiny, 1.5f, INFINITY};
  const float shuffled[8] = {0.0f, INFINITY, -tiny, 1.5f, -0.0f, -INFINITY, tiny, -1.5f};
  thrust::device_vector<float> d(shuffled, shuffled + 8);
  thrust::sort(d.begin(), d.end());
  thrust::host_vector<float> got(d);
  ASSERT_TRUE(std::memcmp(got.data(), ordered, sizeof(ordered)) == 0);
}
DECLARE_UNITTEST(TestSortFloatKeys);

// testing/sort_by_key.cu:46-85
template <class T>
void TestSortByKeySimple() {
  const T keys[7] = {1, 3, 6, 5, 2, 0, 4};
  const T vals[7] = {0, 1, 2, 3, 4, 5, 6};
  const T sorted_vals[7] = {5, 0, 4, 1, 6, 3, 2};
  thrust::device_vector<T> dk(keys, keys + 7), dv(vals, vals + 7);
  thrust::sort_by_key(dk.begin(), dk.end(), dv.begin());
  thrust::host_vector<T> ek(7), ev(sorted_vals, sorted_vals + 7);
  for (int i = 0; i < 7; i++) ek[i] = (T)i;
  ASSERT_EQUAL(dk, ek);
  ASSERT_EQUAL(dv, ev);
}
DECLARE_TYPED_UNITTEST(TestSortByKeySimple, int);
DECLARE_TYPED_UNITTEST(TestSortByKeySimple, uint8_t);
DECLARE_TYPED_UNITTEST(TestSortByKeySimple, int64_t);
DECLARE_TYPED_UNITTEST(TestSortByKeySimple, float);

// testing/sort_by_key.cu:88-103 and stable_sort_by_key.cu:98-116: many duplicate keys, values
// are the original positions, so any instability shows
template <class K>
void TestStableSortByKey() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<K> hk = unittest::random_integers<K>(n);
    for (std::size_t i = 0; i < n; i++) hk[i] = (K)(hk[i] % 29);
    thrust::host_vector<uint32_t> hv(n);
    for (std::size_t i = 0; i < n; i++) hv[i] = (uint32_t)i;
    thrust::device_vector<K> dk = hk;
    thrust::device_vector<uint32_t> dv = hv;
    thrust::stable_sort_by_key(hk.begin(), hk.end(), hv.begin());
    thrust::stable_sort_by_key(dk.begin(), dk.end(), dv.begin());
    ASSERT_EQUAL(hk, dk);
    ASSERT_EQUAL(hv, dv);
    // descending keeps the input order of equal keys too (thrust.example.sort.filecheck:19-21)
    thrust::stable_sort_by_key(hk.begin(), hk.end(), hv.begin(), thrust::greater<K>());
    thrust::stable_sort_by_key(dk.begin(), dk.end(), dv.begin(), thrust::greater<K>());
    ASSERT_EQUAL(hk, dk);
    ASSERT_EQUAL(hv, dv);
  }
}
DECLARE_TYPED_UNITTEST(TestStableSortByKey, int);
DECLARE_TYPED_UNITTEST(TestStableSortByKey, uint64_t);
DECLARE_TYPED_UNITTEST(TestStableSortByKey, uint8_t);

// internal/test/thrust.example.sort.filecheck:16-21
void TestSortExampleGolden() {
  const int keys[16] = {79, 78, 62, 78, 94, 40, 86, 57, 40, 16, 28, 54, 77, 87, 93, 98};
  const int asc_k[16] = {16, 28, 40, 40, 54, 57, 62, 77, 78, 78, 79, 86, 87, 93, 94, 98};
  const int asc_v[16] = {9, 10, 5, 8, 11, 7, 2, 12, 1, 3, 0, 6, 13, 14, 4, 15};
  const int desc_v[16] = {15, 4, 14, 13, 6, 0, 1, 3, 12, 2, 7, 11, 5, 8, 10, 9};
  thrust::device_vector<int> k(keys, keys + 16), v(16);
  for (int i = 0; i < 16; i++) v[i] = i;
  thrust::sort_by_key(k.begin(), k.end(), v.begin());
  ASSERT_EQUAL(k, thrust::host_vector<int>(asc_k, asc_k + 16));
  ASSERT_EQUAL(v, thrust::host_vector<int>(asc_v, asc_v + 16));
  k = thrust::host_vector<int>(keys, keys + 16);
  for (int i = 0; i < 16; i++) v[i] = i;
  thrust::sort_by_key(k.begin(), k.end(), v.begin(), thrust::greater<int>());
  ASSERT_EQUAL(v, thrust::host_vector<int>(desc_v, desc_v + 16));
}
DECLARE_UNITTEST(TestSortExampleGolden);

// testing/sort_variable_bits.cu:17-43
void TestSortVariableBits() {
  const std::size_t n = 20011;
  for (int bits = 0; bits < 32; bits += 3) {
    thrust::host_vector<uint32_t> h = unittest::random_integers<uint32_t>(n, bits);
    const uint32_t mask = (1u << bits) - 1;
    for (auto& x : h) x &= mask;
    thrust::device_vector<uint32_t> d = h;
    std::sort(h.begin(), h.end());
    thrust::sort(d.begin(), d.end());
    ASSERT_EQUAL(h, d);
  }
}
DECLARE_UNITTEST(TestSortVariableBits);

// raw device pointers under an explicit policy, and an unaligned sub-range
void TestSortRawPointersAndSubrange() {
  thrust::host_vector<int> h = unittest::random_integers<int>(10007);
  thrust::device_vector<int> d = h;
  int* raw = thrust::raw_pointer_cast(d.data());
  thrust::sort(thrust::device, raw + 3, raw + 10007);
  std::sort(h.begin() + 3, h.end());
  ASSERT_EQUAL(h, d);
}
DECLARE_UNITTEST(TestSortRawPointersAndSubrange);

// Floating-point keys: host and device ranges give the same order bit for bit — the total order of
// the reference's radix encoding (thrust/system/detail/sequential/stable_radix_sort.inl:43-139):
// -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN, equal keys in input order; descending is the
// stable mirror image.
template <class T, class U>
void TestSortFloatTotalOrderHostAndDevice() {
  const T nan = std::numeric_limits<T>::quiet_NaN(), inf = std::numeric_limits<T>::infinity(), tiny = std::numeric_limits<T>::denorm_min();
  const T specials[] = {T(0), -T(0), nan, -nan, inf, -inf, tiny, -tiny, T(1), T(-1)};
  const std::size_t n = 100000;
  thrust::host_vector<T> h(n);
  std::uint64_t s = 5;
  for (std::size_t i = 0; i < n; i++) {
    const std::uint64_t r = unittest::splitmix64(s);
    h[i] = (r & 3) == 0 ? specials[(r >> 2) % 10] : (T)((double)(r >> 11) / 9007199254740992.0 * 8.0 - 4.0);
  }
  thrust::host_vector<int> hv(n);
  for (std::size_t i = 0; i < n; i++) hv[i] = (int)i;
  auto bits = [](const thrust::host_vector<T>& v) {
    thrust::host_vector<U> b(v.size());
    std::memcpy(b.data(), v.data(), v.size() * sizeof(T));
    return b;
  };
  for (int descending = 0; descending < 2; descending++) {
    thrust::host_vector<T> hk = h;
    thrust::host_vector<int> hvals = hv;
    thrust::device_vector<T> dk = h;
    thrust::device_vector<int> dvals = hv;
    if (descending) {
      thrust::sort_by_key(hk.begin(), hk.end(), hvals.begin(), thrust::greater<T>());
      thrust::sort_by_key(dk.begin(), dk.end(), dvals.begin(), thrust::greater<T>());
    } else {
      thrust::sort_by_key(hk.begin(), hk.end(), hvals.begin());
      thrust::sort_by_key(dk.begin(), dk.end(), dvals.begin());
    }
    ASSERT_EQUAL(bits(thrust::host_vector<T>(dk)), bits(hk));
    ASSERT_EQUAL(dvals, hvals);
    thrust::host_vector<T> hs = h;
    thrust::device_vector<T> ds = h;
    if (descending) {
      thrust::sort(hs.begin(), hs.end(), thrust::greater<T>());
      thrust::sort(ds.begin(), ds.end(), thrust::greater<T>());
    } else {
      thrust::sort(hs.begin(), hs.end());
      thrust::sort(ds.begin(), ds.end());
    }
    ASSERT_EQUAL(bits(thrust::host_vector<T>(ds)), bits(hs));
    ASSERT_TRUE(std::signbit(hs[descending ? n - 1 : 0]) && std::isnan(hs[descending ? n - 1 : 0]));  // -NaN at the low end
  }
}
void TestSortFloatTotalOrder() {
  TestSortFloatTotalOrderHostAndDevice<float, std::uint32_t>();
  TestSortFloatTotalOrderHostAndDevice<double, std::uint64_t>();
}
DECLARE_UNITTEST(TestSortFloatTotalOrder);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
