// merge / merge_by_key and the set operations on device ranges: the reference's known answers
// (testing/merge.cu:12-40, merge_by_key.cu:10-45, set_union.cu:70-115, set_intersection.cu:70-95,
// set_difference.cu:70-95, set_symmetric_difference.cu:70-95 and the _by_key files :85-120), then
// device against the sequential algorithm on host ranges over the size ladder — sorted inputs with
// many duplicates, so that the multiset rules and the order of equivalent elements are exercised.
#include <thrust/functional.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/merge.h>
#include <thrust/set_operations.h>
#include <thrust/sort.h>

#include <algorithm>

#include "testing.h"

template <class T>
thrust::host_vector<T> hv(std::initializer_list<double> v) {
  thrust::host_vector<T> r;
  for (double x : v) r.push_back((T)x);
  return r;
}
// n sorted values drawn from [0, range)
template <class T>
thrust::host_vector<T> sorted_values(std::size_t n, std::uint64_t seed, std::uint64_t range) {
  thrust::host_vector<T> v(n);
  std::uint64_t s = seed * 7919 + n;
  for (auto& x : v) x = (T)(unittest::splitmix64(s) % range);
  std::sort(v.begin(), v.end());
  return v;
}

void TestMergeSimple() {
  thrust::device_vector<int> a = hv<int>({0, 2, 4}), b = hv<int>({0, 3, 3, 4}), out(7);
  auto end = thrust::merge(a.begin(), a.end(), b.begin(), b.end(), out.begin());
  ASSERT_EQUAL(end - out.begin(), 7);
  ASSERT_EQUAL(out, hv<int>({0, 0, 2, 3, 3, 4, 4}));
  thrust::device_vector<int> av = hv<int>({13, 7, 42}), bv = hv<int>({42, 42, 7, 13}), ko(7), vo(7);
  auto ends = thrust::merge_by_key(a.begin(), a.end(), b.begin(), b.end(), av.begin(), bv.begin(), ko.begin(), vo.begin());
  ASSERT_EQUAL(ends.first - ko.begin(), 7);
  ASSERT_EQUAL(ends.second - vo.begin(), 7);
  ASSERT_EQUAL(ko, hv<int>({0, 0, 2, 3, 3, 4, 4}));
  ASSERT_EQUAL(vo, hv<int>({13, 42, 7, 42, 7, 42, 13}));  // of equal keys the first range's value comes first
  // descending ranges under greater
  thrust::device_vector<int> c = hv<int>({9, 5, 5, 1}), d = hv<int>({7, 5, 0}), o2(7);
  thrust::merge(c.begin(), c.end(), d.begin(), d.end(), o2.begin(), thrust::greater<int>());
  ASSERT_EQUAL(o2, hv<int>({9, 7, 5, 5, 5, 1, 0}));
  // an empty range on either side
  thrust::device_vector<int> none, o3(3);
  ASSERT_EQUAL(thrust::merge(a.begin(), a.end(), none.begin(), none.end(), o3.begin()) - o3.begin(), 3);
  ASSERT_EQUAL(o3, hv<int>({0, 2, 4}));
  ASSERT_EQUAL(thrust::merge(none.begin(), none.end(), a.begin(), a.end(), o3.begin()) - o3.begin(), 3);
  ASSERT_EQUAL(o3, hv<int>({0, 2, 4}));
  ASSERT_EQUAL(thrust::merge(none.begin(), none.end(), none.begin(), none.end(), o3.begin()) - o3.begin(), 0);
}
DECLARE_UNITTEST(TestMergeSimple);

void TestSetOperationsSimple() {
  {
    thrust::device_vector<int> a = hv<int>({0, 2, 4}), b = hv<int>({0, 3, 3, 4}), out(5);
    ASSERT_EQUAL(thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), out.begin()) - out.begin(), 5);
    ASSERT_EQUAL(out, hv<int>({0, 2, 3, 3, 4}));
    thrust::device_vector<int> a2 = hv<int>({0, 2, 2}), b2 = hv<int>({0, 2, 2, 2, 3});  // duplicates: max(m, n) of each
    ASSERT_EQUAL(thrust::set_union(a2.begin(), a2.end(), b2.begin(), b2.end(), out.begin()) - out.begin(), 5);
    ASSERT_EQUAL(out, hv<int>({0, 2, 2, 2, 3}));
    thrust::device_vector<int> o2(2);
    ASSERT_EQUAL(thrust::set_intersection(a.begin(), a.end(), b.begin(), b.end(), o2.begin()) - o2.begin(), 2);
    ASSERT_EQUAL(o2, hv<int>({0, 4}));
  }
  {
    thrust::device_vector<int> a = hv<int>({0, 2, 4, 5}), b = hv<int>({0, 3, 3, 4, 6}), out(2);
    ASSERT_EQUAL(thrust::set_difference(a.begin(), a.end(), b.begin(), b.end(), out.begin()) - out.begin(), 2);
    ASSERT_EQUAL(out, hv<int>({2, 5}));
  }
  {
    thrust::device_vector<int> a = hv<int>({0, 2, 4, 6}), b = hv<int>({0, 3, 3, 4, 7}), out(5);
    ASSERT_EQUAL(thrust::set_symmetric_difference(a.begin(), a.end(), b.begin(), b.end(), out.begin()) - out.begin(), 5);
    ASSERT_EQUAL(out, hv<int>({2, 3, 3, 6, 7}));
  }
}
DECLARE_UNITTEST(TestSetOperationsSimple);

void TestSetOperationsByKeySimple() {
  thrust::device_vector<int> ak = hv<int>({0, 2, 4}), av = hv<int>({0, 0, 0}), bk = hv<int>({0, 3, 3, 4}), bv = hv<int>({1, 1, 1, 1});
  {
    thrust::device_vector<int> ko(5), vo(5);
    auto e = thrust::set_union_by_key(ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(), bv.begin(), ko.begin(), vo.begin());
    ASSERT_EQUAL(e.first - ko.begin(), 5);
    ASSERT_EQUAL(ko, hv<int>({0, 2, 3, 3, 4}));
    ASSERT_EQUAL(vo, hv<int>({0, 0, 1, 1, 0}));
  }
  {
    thrust::device_vector<int> ko(2), vo(2);
    auto e = thrust::set_intersection_by_key(ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(), ko.begin(), vo.begin());
    ASSERT_EQUAL(e.first - ko.begin(), 2);
    ASSERT_EQUAL(ko, hv<int>({0, 4}));
    ASSERT_EQUAL(vo, hv<int>({0, 0}));
  }
  {
    thrust::device_vector<int> ak2 = hv<int>({0, 2, 4, 5}), av2(4, 0), bk2 = hv<int>({0, 3, 3, 4, 6}), bv2(5, 1), ko(2), vo(2);
    auto e = thrust::set_difference_by_key(ak2.begin(), ak2.end(), bk2.begin(), bk2.end(), av2.begin(), bv2.begin(), ko.begin(), vo.begin());
    ASSERT_EQUAL(e.first - ko.begin(), 2);
    ASSERT_EQUAL(ko, hv<int>({2, 5}));
    ASSERT_EQUAL(vo, hv<int>({0, 0}));
  }
  {
    thrust::device_vector<int> ak2 = hv<int>({0, 2, 4, 6}), av2(4, 0), bk2 = hv<int>({0, 3, 3, 4, 7}), bv2(5, 1), ko(5), vo(5);
    auto e = thrust::set_symmetric_difference_by_key(ak2.begin(), ak2.end(), bk2.begin(), bk2.end(), av2.begin(), bv2.begin(), ko.begin(), vo.begin());
    ASSERT_EQUAL(e.first - ko.begin(), 5);
    ASSERT_EQUAL(ko, hv<int>({2, 3, 3, 6, 7}));
    ASSERT_EQUAL(vo, hv<int>({0, 1, 1, 0, 1}));
  }
}
DECLARE_UNITTEST(TestSetOperationsByKeySimple);

// device vs the sequential algorithm; ranges of different lengths, heavy duplication
template <class T>
void TestMergeAndSetOperationsLadder() {
  for (std::size_t n : unittest::sizes()) {
    if (n > 200000 && sizeof(T) == 1) continue;
    const std::size_t nb = n / 3 * 2 + (n % 5);
    const std::uint64_t range = sizeof(T) == 1 ? 100 : (n / 4 + 3);
    thrust::host_vector<T> ha = sorted_values<T>(n, 1, range), hb = sorted_values<T>(nb, 2, range);
    thrust::device_vector<T> da = ha, db = hb;
    thrust::host_vector<T> ho(n + nb);
    thrust::device_vector<T> dout(n + nb);
    {
      auto he = thrust::merge(ha.begin(), ha.end(), hb.begin(), hb.end(), ho.begin());
      auto de = thrust::merge(da.begin(), da.end(), db.begin(), db.end(), dout.begin());
      ASSERT_EQUAL(de - dout.begin(), he - ho.begin());
      ASSERT_EQUAL(dout, ho);
    }
#define CHECK_SET(NAME)                                                                       \
  {                                                                                           \
    auto he = thrust::NAME(ha.begin(), ha.end(), hb.begin(), hb.end(), ho.begin());           \
    auto de = thrust::NAME(da.begin(), da.end(), db.begin(), db.end(), dout.begin());         \
    ASSERT_EQUAL(de - dout.begin(), he - ho.begin());                                         \
    thrust::host_vector<T> got(dout.begin(), de), want(ho.begin(), he);                       \
    ASSERT_EQUAL(got, want);                                                                  \
    auto se = std::NAME(ha.begin(), ha.end(), hb.begin(), hb.end(), ho.begin());              \
    ASSERT_EQUAL(se - ho.begin(), he - ho.begin()); /* and the host path equals the standard's */ \
  }
    CHECK_SET(set_union)
    CHECK_SET(set_intersection)
    CHECK_SET(set_difference)
    CHECK_SET(set_symmetric_difference)
#undef CHECK_SET
  }
}
DECLARE_TYPED_UNITTEST(TestMergeAndSetOperationsLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestMergeAndSetOperationsLadder, uint8_t);
DECLARE_TYPED_UNITTEST(TestMergeAndSetOperationsLadder, int64_t);
DECLARE_TYPED_UNITTEST(TestMergeAndSetOperationsLadder, double);

// values are the positions in their range (+ a mark for the second range): the test sees which
// range each result came from and that equal keys keep their order
void TestByKeyLadder() {
  for (std::size_t n : unittest::sizes()) {
    const std::size_t nb = n / 2 + 7;
    thrust::host_vector<int> hak = sorted_values<int>(n, 3, n / 3 + 2), hbk = sorted_values<int>(nb, 4, n / 3 + 2);
    thrust::host_vector<int> hav(n), hbv(nb);
    for (std::size_t i = 0; i < n; i++) hav[i] = (int)i;
    for (std::size_t i = 0; i < nb; i++) hbv[i] = (int)(i + (1u << 30));
    thrust::device_vector<int> dak = hak, dbk = hbk, dav = hav, dbv = hbv;
    thrust::host_vector<int> hko(n + nb), hvo(n + nb);
    thrust::device_vector<int> dko(n + nb), dvo(n + nb);
    {
      auto he = thrust::merge_by_key(hak.begin(), hak.end(), hbk.begin(), hbk.end(), hav.begin(), hbv.begin(), hko.begin(), hvo.begin());
      auto de = thrust::merge_by_key(dak.begin(), dak.end(), dbk.begin(), dbk.end(), dav.begin(), dbv.begin(), dko.begin(), dvo.begin());
      ASSERT_EQUAL(de.first - dko.begin(), he.first - hko.begin());
      ASSERT_EQUAL(dko, hko);
      ASSERT_EQUAL(dvo, hvo);
    }
#define CHECK_BY_KEY(NAME)                                                                                                              \
  {                                                                                                                                     \
    auto he = thrust::NAME(hak.begin(), hak.end(), hbk.begin(), hbk.end(), hav.begin(), hbv.begin(), hko.begin(), hvo.begin());         \
    auto de = thrust::NAME(dak.begin(), dak.end(), dbk.begin(), dbk.end(), dav.begin(), dbv.begin(), dko.begin(), dvo.begin());         \
    ASSERT_EQUAL(de.first - dko.begin(), he.first - hko.begin());                                                                       \
    ASSERT_EQUAL(de.second - dvo.begin(), he.second - hvo.begin());                                                                     \
    ASSERT_EQUAL(thrust::host_vector<int>(dko.begin(), de.first), thrust::host_vector<int>(hko.begin(), he.first));                     \
    ASSERT_EQUAL(thrust::host_vector<int>(dvo.begin(), de.second), thrust::host_vector<int>(hvo.begin(), he.second));                   \
  }
    CHECK_BY_KEY(set_union_by_key)
    CHECK_BY_KEY(set_difference_by_key)
    CHECK_BY_KEY(set_symmetric_difference_by_key)
#undef CHECK_BY_KEY
    {
      auto he = thrust::set_intersection_by_key(hak.begin(), hak.end(), hbk.begin(), hbk.end(), hav.begin(), hko.begin(), hvo.begin());
      auto de = thrust::set_intersection_by_key(dak.begin(), dak.end(), dbk.begin(), dbk.end(), dav.begin(), dko.begin(), dvo.begin());
      ASSERT_EQUAL(de.first - dko.begin(), he.first - hko.begin());
      ASSERT_EQUAL(thrust::host_vector<int>(dko.begin(), de.first), thrust::host_vector<int>(hko.begin(), he.first));
      ASSERT_EQUAL(thrust::host_vector<int>(dvo.begin(), de.second), thrust::host_vector<int>(hvo.begin(), he.second));
    }
  }
}
DECLARE_UNITTEST(TestByKeyLadder);

// fancy iterators in and out, a user comparison on a struct, an explicit policy
struct point {
  int x, y;
  __host__ __device__ bool operator==(const point& o) const { return x == o.x && y == o.y; }
};
std::ostream& operator<<(std::ostream& os, const point& p) { return os << "(" << p.x << "," << p.y << ")"; }
struct by_x {
  __host__ __device__ bool operator()(const point& a, const point& b) const { return a.x < b.x; }
};
void TestMergeFancyAndStructs() {
  // evens merged with a counting range: every number once or twice
  thrust::device_vector<int> evens = hv<int>({0, 2, 4, 6, 8}), out(15);
  thrust::merge(thrust::device, evens.begin(), evens.end(), thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(10), out.begin());
  ASSERT_EQUAL(out, hv<int>({0, 0, 1, 2, 2, 3, 4, 4, 5, 6, 6, 7, 8, 8, 9}));
  // the intersection of two counting ranges, result count only
  auto e = thrust::set_intersection(thrust::device, thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(1000),
                                    thrust::counting_iterator<int>(500), thrust::counting_iterator<int>(2000), thrust::make_discard_iterator());
  ASSERT_EQUAL(e - thrust::make_discard_iterator(), 500);
  // structs ordered by one member: equivalent elements keep the first range first and their own order
  const std::size_t n = 5000;
  thrust::host_vector<point> ha(n), hb(n), ho(2 * n);
  for (std::size_t i = 0; i < n; i++) {
    ha[i] = point{(int)(i / 7), (int)i};
    hb[i] = point{(int)(i / 5), (int)(i + 100000)};
  }
  thrust::device_vector<point> da = ha, db = hb, dout(2 * n);
  thrust::merge(ha.begin(), ha.end(), hb.begin(), hb.end(), ho.begin(), by_x());
  thrust::merge(da.begin(), da.end(), db.begin(), db.end(), dout.begin(), by_x());
  ASSERT_EQUAL(dout, ho);
  auto he = thrust::set_difference(hb.begin(), hb.end(), ha.begin(), ha.end(), ho.begin(), by_x());
  auto de = thrust::set_difference(db.begin(), db.end(), da.begin(), da.end(), dout.begin(), by_x());
  ASSERT_EQUAL(de - dout.begin(), he - ho.begin());
  ASSERT_EQUAL(thrust::host_vector<point>(dout.begin(), de), thrust::host_vector<point>(ho.begin(), he));
}
DECLARE_UNITTEST(TestMergeFancyAndStructs);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
