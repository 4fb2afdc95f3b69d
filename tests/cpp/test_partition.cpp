// partition / stable_partition / partition_copy with user predicates, in the shape of the
// reference's testing/partition.cu: its known answers plus device vs host over the size ladder.
// Compiled by hipcc (the predicates instantiate kernel templates).
#include <algorithm>

#include <thrust/functional.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/partition.h>
#include <thrust/remove.h>
#include <thrust/tuple.h>
#include <thrust/sequence.h>

#include "testing.h"

template <class T>
struct is_even {
  __host__ __device__ bool operator()(T x) const { return ((int)x % 2) == 0; }
};

template <class T>
thrust::host_vector<T> vec(std::initializer_list<int> l) {
  thrust::host_vector<T> h(l.size());
  std::size_t i = 0;
  for (int x : l) h[i++] = (T)x;
  return h;
}

// testing/partition.cu:25-59, :63-93
template <class T>
void TestPartitionSimple() {
  thrust::device_vector<T> data = vec<T>({1, 2, 1, 1, 2});
  auto iter = thrust::partition(data.begin(), data.end(), is_even<T>());
  ASSERT_EQUAL(iter - data.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(data, vec<T>({2, 2, 1, 1, 1}));
  data = vec<T>({0, 1, 0, 0, 1});
  thrust::device_vector<T> stencil = vec<T>({1, 2, 1, 1, 2});
  iter = thrust::partition(data.begin(), data.end(), stencil.begin(), is_even<T>());
  ASSERT_EQUAL(iter - data.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(data, vec<T>({1, 1, 0, 0, 0}));
}
DECLARE_TYPED_UNITTEST(TestPartitionSimple, int);
DECLARE_TYPED_UNITTEST(TestPartitionSimple, int8_t);
DECLARE_TYPED_UNITTEST(TestPartitionSimple, int16_t);

// testing/partition.cu:98-128, :133-170
template <class T>
void TestPartitionCopySimple() {
  thrust::device_vector<T> data = vec<T>({1, 2, 1, 1, 2}), yes(2), no(3);
  auto ends = thrust::partition_copy(data.begin(), data.end(), yes.begin(), no.begin(), is_even<T>());
  ASSERT_EQUAL(ends.first - yes.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(ends.second - no.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(yes, vec<T>({2, 2}));
  ASSERT_EQUAL(no, vec<T>({1, 1, 1}));
  data = vec<T>({0, 1, 0, 0, 1});
  thrust::device_vector<T> stencil = vec<T>({1, 2, 1, 1, 2});
  ends = thrust::partition_copy(thrust::device, data.begin(), data.end(), stencil.begin(), yes.begin(), no.begin(), is_even<T>());
  ASSERT_EQUAL(ends.first - yes.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(ends.second - no.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(yes, vec<T>({1, 1}));
  ASSERT_EQUAL(no, vec<T>({0, 0, 0}));
}
DECLARE_TYPED_UNITTEST(TestPartitionCopySimple, int);
DECLARE_TYPED_UNITTEST(TestPartitionCopySimple, int8_t);

// testing/partition.cu:175-198, :203-233, :238-268, :273-310
template <class T>
void TestStablePartitionSimple() {
  thrust::device_vector<T> data = vec<T>({1, 2, 1, 3, 2});
  auto iter = thrust::stable_partition(data.begin(), data.end(), is_even<T>());
  ASSERT_EQUAL(iter - data.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(data, vec<T>({2, 2, 1, 1, 3}));
  data = vec<T>({1, 2, 1, 3, 2});
  thrust::device_vector<T> stencil = vec<T>({0, 1, 0, 0, 1});  // odd stencil entries are rejected
  iter = thrust::stable_partition(data.begin(), data.end(), stencil.begin(), is_even<T>());
  ASSERT_EQUAL(iter - data.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(data, vec<T>({1, 1, 3, 2, 2}));
  data = vec<T>({1, 2, 1, 3, 2});
  iter = thrust::stable_partition(data.begin(), data.end(), stencil.begin(), thrust::identity<T>());
  ASSERT_EQUAL(iter - data.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(data, vec<T>({2, 2, 1, 1, 3}));
  data = vec<T>({1, 2, 1, 1, 2});
  thrust::device_vector<T> yes(2), no(3);
  auto ends = thrust::stable_partition_copy(data.begin(), data.end(), yes.begin(), no.begin(), is_even<T>());
  ASSERT_EQUAL(ends.first - yes.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(ends.second - no.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(yes, vec<T>({2, 2}));
  ASSERT_EQUAL(no, vec<T>({1, 1, 1}));
}
DECLARE_TYPED_UNITTEST(TestStablePartitionSimple, int);
DECLARE_TYPED_UNITTEST(TestStablePartitionSimple, int64_t);
DECLARE_TYPED_UNITTEST(TestStablePartitionSimple, uint8_t);

// testing/partition.cu:315-335, :719-741: in place over the ladder, against std::stable_partition
template <class T>
void TestStablePartition() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    thrust::device_vector<T> d = h;
    auto hi = thrust::stable_partition(h.begin(), h.end(), is_even<T>());
    auto di = thrust::stable_partition(d.begin(), d.end(), is_even<T>());
    ASSERT_EQUAL(hi - h.begin(), di - d.begin());
    ASSERT_EQUAL(h, d);
  }
}
DECLARE_TYPED_UNITTEST(TestStablePartition, int);
DECLARE_TYPED_UNITTEST(TestStablePartition, int8_t);
DECLARE_TYPED_UNITTEST(TestStablePartition, int64_t);

// testing/partition.cu:337-370, :743-764: with a stencil of another type
template <class T>
void TestStablePartitionStencil() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h(n);
    thrust::sequence(h.begin(), h.end());
    thrust::host_vector<uint16_t> hs = unittest::random_integers<uint16_t>(n);
    thrust::device_vector<T> d = h;
    thrust::device_vector<uint16_t> ds = hs;
    auto hi = thrust::stable_partition(h.begin(), h.end(), hs.begin(), is_even<uint16_t>());
    auto di = thrust::stable_partition(d.begin(), d.end(), ds.begin(), is_even<uint16_t>());
    ASSERT_EQUAL(hi - h.begin(), di - d.begin());
    ASSERT_EQUAL(h, d);
    ASSERT_EQUAL(hs, ds);
  }
}
DECLARE_TYPED_UNITTEST(TestStablePartitionStencil, int);
DECLARE_TYPED_UNITTEST(TestStablePartitionStencil, double);

// testing/partition.cu:372-412, :766-802
template <class T>
void TestPartitionCopy() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n), hy(n), hn(n);
    thrust::device_vector<T> d = h, dy(n), dn(n);
    auto he = thrust::partition_copy(h.begin(), h.end(), hy.begin(), hn.begin(), is_even<T>());
    auto de = thrust::partition_copy(d.begin(), d.end(), dy.begin(), dn.begin(), is_even<T>());
    ASSERT_EQUAL(he.first - hy.begin(), de.first - dy.begin());
    ASSERT_EQUAL(he.second - hn.begin(), de.second - dn.begin());
    ASSERT_EQUAL((he.first - hy.begin()) + (he.second - hn.begin()), (std::ptrdiff_t)n);
    hy.resize(he.first - hy.begin()); dy.resize(hy.size());
    hn.resize(he.second - hn.begin()); dn.resize(hn.size());
    ASSERT_EQUAL(hy, dy);
    ASSERT_EQUAL(hn, dn);
    ASSERT_EQUAL(d, h);
  }
}
DECLARE_TYPED_UNITTEST(TestPartitionCopy, int);
DECLARE_TYPED_UNITTEST(TestPartitionCopy, int16_t);
DECLARE_TYPED_UNITTEST(TestPartitionCopy, uint64_t);

// 2^25 + 5 elements: many tiles, the rejected positions span the look-back chain
void TestStablePartitionLarge() {
  const std::size_t n = (std::size_t(1) << 25) + 5;
  thrust::host_vector<int> h = unittest::random_integers<int>(n);
  thrust::device_vector<int> d = h;
  auto hi = std::stable_partition(h.begin(), h.end(), is_even<int>());
  auto di = thrust::stable_partition(d.begin(), d.end(), is_even<int>());
  ASSERT_EQUAL(hi - h.begin(), di - d.begin());
  ASSERT_EQUAL(h, d);
}
DECLARE_UNITTEST(TestStablePartitionLarge);

// testing/partition.cu:760-860 (TestPartitionZipIterator, TestStablePartitionZipIterator) and
// testing/remove.cu: in place over a zipped pair of device arrays, with and without a stencil;
// remove_if / remove_copy_if with a stencil and remove_copy of a value
struct first_is_even {
  __host__ __device__ bool operator()(const thrust::tuple<int, int>& t) const { return (thrust::get<0>(t) & 1) == 0; }
};
struct is_odd_int { __host__ __device__ bool operator()(int x) const { return (x & 1) != 0; } };
void TestPartitionAndRemoveOverZippedRanges() {
  for (std::size_t n : {std::size_t(0), std::size_t(1), std::size_t(5), std::size_t(1000), std::size_t(70001)}) {
    thrust::host_vector<int> ha(n), hb(n), hs(n);
    for (std::size_t i = 0; i < n; i++) { ha[i] = (int)((i * 2654435761u) >> 7) % 1000; hb[i] = (int)i; hs[i] = (int)(i % 3); }
    std::vector<std::pair<int, int>> ref(n);
    for (std::size_t i = 0; i < n; i++) ref[i] = {ha[i], hb[i]};
    {  // stable_partition of zip(a, b) by a's parity
      thrust::device_vector<int> a = ha, b = hb;
      auto zb = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin()));
      auto mid = thrust::stable_partition(zb, zb + n, first_is_even());
      auto r = ref;
      auto rm = std::stable_partition(r.begin(), r.end(), [](const std::pair<int, int>& p) { return (p.first & 1) == 0; });
      ASSERT_EQUAL((std::size_t)(mid - zb), (std::size_t)(rm - r.begin()));
      thrust::host_vector<int> ra(n), rb(n);
      for (std::size_t i = 0; i < n; i++) { ra[i] = r[i].first; rb[i] = r[i].second; }
      ASSERT_EQUAL(a, ra);
      ASSERT_EQUAL(b, rb);
    }
    {  // the same with a stencil: element i is accepted when stencil[i] is odd
      thrust::device_vector<int> a = ha, b = hb, st = hs;
      auto zb = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin()));
      auto mid = thrust::stable_partition(zb, zb + n, st.begin(), is_odd_int());
      thrust::host_vector<int> ra, rb;
      for (std::size_t i = 0; i < n; i++) if (hs[i] & 1) { ra.push_back(ha[i]); rb.push_back(hb[i]); }
      const std::size_t c = ra.size();
      for (std::size_t i = 0; i < n; i++) if (!(hs[i] & 1)) { ra.push_back(ha[i]); rb.push_back(hb[i]); }
      ASSERT_EQUAL((std::size_t)(mid - zb), c);
      ASSERT_EQUAL(a, ra);
      ASSERT_EQUAL(b, rb);
    }
    {  // remove_if over the zip
      thrust::device_vector<int> a = ha, b = hb;
      auto zb = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin()));
      auto end = thrust::remove_if(zb, zb + n, first_is_even());
      thrust::host_vector<int> ra, rb;
      for (std::size_t i = 0; i < n; i++) if (ha[i] & 1) { ra.push_back(ha[i]); rb.push_back(hb[i]); }
      ASSERT_EQUAL((std::size_t)(end - zb), ra.size());
      a.resize(ra.size()); b.resize(rb.size());
      ASSERT_EQUAL(a, ra);
      ASSERT_EQUAL(b, rb);
    }
    {  // remove_if and remove_copy_if with a stencil, remove_copy of a value
      thrust::device_vector<int> a = ha, st = hs, out(n), out2(n);
      auto e1 = thrust::remove_copy_if(a.begin(), a.end(), st.begin(), out.begin(), is_odd_int());
      auto e2 = thrust::remove_copy(a.begin(), a.end(), out2.begin(), n ? ha[0] : 0);
      auto e0 = thrust::remove_if(a.begin(), a.end(), st.begin(), is_odd_int());
      thrust::host_vector<int> r1, r2;
      for (std::size_t i = 0; i < n; i++) { if (!(hs[i] & 1)) r1.push_back(ha[i]); if (ha[i] != ha[0]) r2.push_back(ha[i]); }
      ASSERT_EQUAL((std::size_t)(e1 - out.begin()), r1.size());
      ASSERT_EQUAL((std::size_t)(e0 - a.begin()), r1.size());
      ASSERT_EQUAL((std::size_t)(e2 - out2.begin()), r2.size());
      out.resize(r1.size()); a.resize(r1.size()); out2.resize(r2.size());
      ASSERT_EQUAL(out, r1);
      ASSERT_EQUAL(a, r1);
      ASSERT_EQUAL(out2, r2);
    }
  }
}
DECLARE_UNITTEST(TestPartitionAndRemoveOverZippedRanges);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
