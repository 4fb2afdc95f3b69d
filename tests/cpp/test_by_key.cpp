// scan_by_key and reduce_by_key tests in the shape of the reference's
// testing/scan_by_key.{inclusive,exclusive}.cu and testing/reduce_by_key.cu.
#include <thrust/functional.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>

#include "testing.h"

template <class T>
thrust::host_vector<T> hv(std::initializer_list<int> v) {
  thrust::host_vector<T> r;
  for (int x : v) r.push_back((T)x);
  return r;
}

// testing/scan_by_key.inclusive.cu:11-75
template <class T>
void TestInclusiveScanByKeySimple() {
  thrust::device_vector<T> keys = hv<T>({0, 1, 1, 1, 2, 3, 3}), vals = hv<T>({1, 2, 3, 4, 5, 6, 7}), out(7, 0);
  auto it = thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin());
  ASSERT_TRUE(it == out.end());
  ASSERT_EQUAL(out, hv<T>({1, 2, 5, 9, 5, 6, 13}));
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin(), thrust::equal_to<T>(),
                                thrust::multiplies<T>());
  ASSERT_EQUAL(out, hv<T>({1, 2, 6, 24, 5, 6, 42}));
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin(), thrust::equal_to<T>());
  ASSERT_EQUAL(out, hv<T>({1, 2, 5, 9, 5, 6, 13}));
}
DECLARE_TYPED_UNITTEST(TestInclusiveScanByKeySimple, int);
DECLARE_TYPED_UNITTEST(TestInclusiveScanByKeySimple, int64_t);
DECLARE_TYPED_UNITTEST(TestInclusiveScanByKeySimple, float);
DECLARE_TYPED_UNITTEST(TestInclusiveScanByKeySimple, uint8_t);

// testing/scan_by_key.exclusive.cu:12-93: init restarts at every segment head
template <class T>
void TestExclusiveScanByKeySimple() {
  thrust::device_vector<T> keys = hv<T>({0, 1, 1, 1, 2, 3, 3}), vals = hv<T>({1, 2, 3, 4, 5, 6, 7}), out(7, 0);
  auto it = thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin());
  ASSERT_TRUE(it == out.end());
  ASSERT_EQUAL(out, hv<T>({0, 0, 2, 5, 0, 0, 6}));
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin(), T(10));
  ASSERT_EQUAL(out, hv<T>({10, 10, 12, 15, 10, 10, 16}));
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin(), T(10), thrust::equal_to<T>(),
                                thrust::multiplies<T>());
  ASSERT_EQUAL(out, hv<T>({10, 10, 20, 60, 10, 10, 60}));
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), out.begin(), T(10), thrust::equal_to<T>());
  ASSERT_EQUAL(out, hv<T>({10, 10, 12, 15, 10, 10, 16}));
}
DECLARE_TYPED_UNITTEST(TestExclusiveScanByKeySimple, int);
DECLARE_TYPED_UNITTEST(TestExclusiveScanByKeySimple, int64_t);
DECLARE_TYPED_UNITTEST(TestExclusiveScanByKeySimple, float);

template <class K>
thrust::host_vector<K> runs_of_keys(std::size_t n, unsigned max_run) {
  thrust::host_vector<K> k(n);
  std::uint64_t s = 4242 + n;
  K cur = 0;
  std::size_t left = 0;
  for (std::size_t i = 0; i < n; i++) {
    if (!left) {
      left = 1 + unittest::splitmix64(s) % max_run;
      cur = (K)(cur + 1 + unittest::splitmix64(s) % 3);
    }
    k[i] = cur;
    --left;
  }
  return k;
}

template <class T>
void TestScanByKey() {
  for (std::size_t n : unittest::sizes()) {
    for (unsigned max_run : {1u, 5u, 700u}) {
      thrust::host_vector<int> hk = runs_of_keys<int>(n, max_run);
      thrust::host_vector<T> hvv = unittest::random_integers<T>(n), ho(n);
      thrust::device_vector<int> dk = hk;
      thrust::device_vector<T> dv = hvv, dout(n);
      thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hvv.begin(), ho.begin());
      thrust::inclusive_scan_by_key(dk.begin(), dk.end(), dv.begin(), dout.begin());
      ASSERT_EQUAL(dout, ho);
      thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hvv.begin(), ho.begin(), (T)7);
      thrust::exclusive_scan_by_key(dk.begin(), dk.end(), dv.begin(), dout.begin(), (T)7);
      ASSERT_EQUAL(dout, ho);
    }
  }
}
DECLARE_TYPED_UNITTEST(TestScanByKey, int);
DECLARE_TYPED_UNITTEST(TestScanByKey, int64_t);
DECLARE_TYPED_UNITTEST(TestScanByKey, uint16_t);

// testing/reduce_by_key.cu:15-112
template <class T>
void TestReduceByKeySimple() {
  thrust::device_vector<T> keys = hv<T>({11, 11, 21, 20, 21, 21, 21, 37, 37});
  thrust::device_vector<T> vals = hv<T>({0, 1, 2, 3, 4, 5, 6, 7, 8});
  thrust::device_vector<T> ok(9), ov(9);
  auto last = thrust::reduce_by_key(keys.begin(), keys.end(), vals.begin(), ok.begin(), ov.begin());
  ASSERT_EQUAL(last.first - ok.begin(), 5);
  ASSERT_EQUAL(last.second - ov.begin(), 5);
  ok.resize(5);
  ov.resize(5);
  ASSERT_EQUAL(ok, hv<T>({11, 21, 20, 21, 37}));
  ASSERT_EQUAL(ov, hv<T>({1, 2, 3, 15, 15}));
  ok.resize(9);
  ov.resize(9);
  last = thrust::reduce_by_key(keys.begin(), keys.end(), vals.begin(), ok.begin(), ov.begin(), thrust::equal_to<T>(),
                               thrust::plus<T>());
  ASSERT_EQUAL(last.first - ok.begin(), 5);
  ok.resize(5);
  ov.resize(5);
  ASSERT_EQUAL(ov, hv<T>({1, 2, 3, 15, 15}));
}
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, int);
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, int64_t);
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, uint8_t);
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, float);

// testing/reduce_by_key.cu:114-156
template <class T>
void TestReduceByKey() {
  for (std::size_t n : unittest::sizes()) {
    for (unsigned max_run : {1u, 9u, 1000u}) {
      thrust::host_vector<int> hk = runs_of_keys<int>(n, max_run);
      thrust::host_vector<T> hvv = unittest::random_integers<T>(n);
      thrust::device_vector<int> dk = hk;
      thrust::device_vector<T> dv = hvv;
      thrust::host_vector<int> hko(n);
      thrust::host_vector<T> hvo(n);
      thrust::device_vector<int> dko(n);
      thrust::device_vector<T> dvo(n);
      auto he = thrust::reduce_by_key(hk.begin(), hk.end(), hvv.begin(), hko.begin(), hvo.begin());
      auto de = thrust::reduce_by_key(dk.begin(), dk.end(), dv.begin(), dko.begin(), dvo.begin());
      ASSERT_EQUAL(he.first - hko.begin(), de.first - dko.begin());
      ASSERT_EQUAL(he.second - hvo.begin(), de.second - dvo.begin());
      const std::size_t r = he.first - hko.begin();
      hko.resize(r); hvo.resize(r); dko.resize(r); dvo.resize(r);
      ASSERT_EQUAL(dko, hko);
      ASSERT_EQUAL(dvo, hvo);
    }
  }
}
DECLARE_TYPED_UNITTEST(TestReduceByKey, int);
DECLARE_TYPED_UNITTEST(TestReduceByKey, int64_t);
DECLARE_TYPED_UNITTEST(TestReduceByKey, uint8_t);

// internal/test/thrust.example.run_length_encoding.filecheck:1-4
void TestRunLengthEncodingExample() {
  const char input[] = "aaabbbbbcddeeeeeeeeeff";
  const std::size_t n = sizeof(input) - 1;
  thrust::device_vector<char> in(input, input + n), out(n);
  thrust::device_vector<int> ones(n, 1), lengths(n);
  auto e = thrust::reduce_by_key(in.begin(), in.end(), ones.begin(), out.begin(), lengths.begin());
  const std::size_t r = e.first - out.begin();
  ASSERT_EQUAL(r, std::size_t(6));
  out.resize(r);
  lengths.resize(r);
  const char ek[] = {'a', 'b', 'c', 'd', 'e', 'f'};
  ASSERT_EQUAL(out, thrust::host_vector<char>(ek, ek + 6));
  ASSERT_EQUAL(lengths, hv<int>({3, 5, 1, 2, 9, 2}));
}
DECLARE_UNITTEST(TestRunLengthEncodingExample);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
