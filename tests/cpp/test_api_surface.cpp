// Every public overload once: with thrust::device, with a stream policy, with thrust::host and
// without a policy on device and host ranges.  Mostly a compile check of the overload sets
// (templates that no other test instantiates); each call's result is also compared between the
// host and the device range.  Compiled by hipcc.
#include <list>
#include <numeric>
#include <sstream>
#include <thrust/adjacent_difference.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/memory.h>
#include <thrust/swap.h>
#include <thrust/universal_vector.h>
#include <thrust/binary_search.h>
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/fill.h>
#include <thrust/for_each.h>
#include <thrust/functional.h>
#include <thrust/partition.h>
#include <thrust/reduce.h>
#include <thrust/remove.h>
#include <thrust/scan.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>
#include <thrust/unique.h>

#include "testing.h"

struct is_odd {
  __host__ __device__ bool operator()(int x) const { return x & 1; }
};
struct plus_one {
  __host__ __device__ void operator()(int& x) const { x += 1; }
};
struct twice {
  __host__ __device__ int operator()(int x) const { return 2 * x; }
};
struct same_half {
  __host__ __device__ bool operator()(int a, int b) const { return a / 2 == b / 2; }
};

typedef thrust::host_vector<int> H;
typedef thrust::device_vector<int> D;

static H input(std::size_t n = 1000) {
  H h = unittest::random_integers<int>(n);
  for (std::size_t i = 0; i < n; i++) h[i] = (int)((unsigned)h[i] % 50);
  return h;
}

// runs the same statement with (policy, range) = (device, D), (stream policy, D), (host, H) and
// without a policy on both; `v` names the range inside the statement, P expands to the policy
#define ON_ALL(STMT_WITH_POLICY, STMT_WITHOUT)                       \
  do {                                                               \
    H hv = input(); D dv = hv;                                       \
    H h0 = hv; D d0 = hv, d1 = hv, d2 = hv; H h1 = hv;               \
    { auto& v = h0; auto P = thrust::host; STMT_WITH_POLICY; }       \
    { auto& v = h1; STMT_WITHOUT; }                                  \
    { auto& v = d0; auto P = thrust::device; STMT_WITH_POLICY; }     \
    { auto& v = d1; auto P = thrust::cdna4::par.on(nullptr); STMT_WITH_POLICY; } \
    { auto& v = d2; STMT_WITHOUT; }                                  \
    ASSERT_EQUAL(h0, h1); ASSERT_EQUAL(h0, d0); ASSERT_EQUAL(h0, d1); ASSERT_EQUAL(h0, d2); \
  } while (0)

void TestSortOverloads() {
  ON_ALL(thrust::sort(P, v.begin(), v.end()), thrust::sort(v.begin(), v.end()));
  ON_ALL(thrust::sort(P, v.begin(), v.end(), thrust::greater<int>()), thrust::sort(v.begin(), v.end(), thrust::greater<int>()));
  ON_ALL(thrust::stable_sort(P, v.begin(), v.end()), thrust::stable_sort(v.begin(), v.end()));
  ON_ALL(thrust::stable_sort(P, v.begin(), v.end(), thrust::less<int>()), thrust::stable_sort(v.begin(), v.end(), thrust::less<int>()));
  ON_ALL({ auto w = v; thrust::sequence(P, w.begin(), w.end()); thrust::sort_by_key(P, v.begin(), v.end(), w.begin()); thrust::transform(P, v.begin(), v.end(), w.begin(), v.begin(), thrust::plus<int>()); },
         { auto w = v; thrust::sequence(w.begin(), w.end()); thrust::sort_by_key(v.begin(), v.end(), w.begin()); thrust::transform(v.begin(), v.end(), w.begin(), v.begin(), thrust::plus<int>()); });
  ON_ALL({ auto w = v; thrust::sequence(P, w.begin(), w.end(), 5); thrust::stable_sort_by_key(P, v.begin(), v.end(), w.begin(), thrust::greater<int>()); thrust::copy(P, w.begin(), w.end(), v.begin()); },
         { auto w = v; thrust::sequence(w.begin(), w.end(), 5); thrust::stable_sort_by_key(v.begin(), v.end(), w.begin(), thrust::greater<int>()); thrust::copy(w.begin(), w.end(), v.begin()); });
}
DECLARE_UNITTEST(TestSortOverloads);

void TestScanOverloads() {
  ON_ALL(thrust::inclusive_scan(P, v.begin(), v.end(), v.begin()), thrust::inclusive_scan(v.begin(), v.end(), v.begin()));
  ON_ALL(thrust::inclusive_scan(P, v.begin(), v.end(), v.begin(), thrust::maximum<int>()), thrust::inclusive_scan(v.begin(), v.end(), v.begin(), thrust::maximum<int>()));
  ON_ALL(thrust::exclusive_scan(P, v.begin(), v.end(), v.begin()), thrust::exclusive_scan(v.begin(), v.end(), v.begin()));
  ON_ALL(thrust::exclusive_scan(P, v.begin(), v.end(), v.begin(), 4), thrust::exclusive_scan(v.begin(), v.end(), v.begin(), 4));
  ON_ALL(thrust::exclusive_scan(P, v.begin(), v.end(), v.begin(), 4, thrust::plus<int>()), thrust::exclusive_scan(v.begin(), v.end(), v.begin(), 4, thrust::plus<int>()));
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); thrust::inclusive_scan_by_key(P, k.begin(), k.end(), v.begin(), v.begin()); },
         { auto k = v; thrust::sort(k.begin(), k.end()); thrust::inclusive_scan_by_key(k.begin(), k.end(), v.begin(), v.begin()); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); thrust::inclusive_scan_by_key(P, k.begin(), k.end(), v.begin(), v.begin(), thrust::equal_to<int>(), thrust::maximum<int>()); },
         { auto k = v; thrust::sort(k.begin(), k.end()); thrust::inclusive_scan_by_key(k.begin(), k.end(), v.begin(), v.begin(), thrust::equal_to<int>(), thrust::maximum<int>()); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); thrust::exclusive_scan_by_key(P, k.begin(), k.end(), v.begin(), v.begin(), 2); },
         { auto k = v; thrust::sort(k.begin(), k.end()); thrust::exclusive_scan_by_key(k.begin(), k.end(), v.begin(), v.begin(), 2); });
}
DECLARE_UNITTEST(TestScanOverloads);

void TestReduceOverloads() {
  ON_ALL(v[0] = thrust::reduce(P, v.begin(), v.end()), v[0] = thrust::reduce(v.begin(), v.end()));
  ON_ALL(v[0] = thrust::reduce(P, v.begin(), v.end(), 7), v[0] = thrust::reduce(v.begin(), v.end(), 7));
  ON_ALL(v[0] = thrust::reduce(P, v.begin(), v.end(), 0, thrust::maximum<int>()), v[0] = thrust::reduce(v.begin(), v.end(), 0, thrust::maximum<int>()));
  ON_ALL(v[0] = thrust::transform_reduce(P, v.begin(), v.end(), twice(), 1, thrust::plus<int>()), v[0] = thrust::transform_reduce(v.begin(), v.end(), twice(), 1, thrust::plus<int>()));
  ON_ALL(v[0] = (int)thrust::count(P, v.begin(), v.end(), 3), v[0] = (int)thrust::count(v.begin(), v.end(), 3));
  ON_ALL(v[0] = (int)thrust::count_if(P, v.begin(), v.end(), is_odd()), v[0] = (int)thrust::count_if(v.begin(), v.end(), is_odd()));
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); auto ko = v; auto vo = v;
           auto e = thrust::reduce_by_key(P, k.begin(), k.end(), v.begin(), ko.begin(), vo.begin());
           thrust::fill(P, v.begin(), v.end(), 0); thrust::copy(P, vo.begin(), e.second, v.begin()); },
         { auto k = v; thrust::sort(k.begin(), k.end()); auto ko = v; auto vo = v;
           auto e = thrust::reduce_by_key(k.begin(), k.end(), v.begin(), ko.begin(), vo.begin());
           thrust::fill(v.begin(), v.end(), 0); thrust::copy(vo.begin(), e.second, v.begin()); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); auto ko = v; auto vo = v;
           auto e = thrust::reduce_by_key(P, k.begin(), k.end(), v.begin(), ko.begin(), vo.begin(), thrust::equal_to<int>(), thrust::maximum<int>());
           thrust::fill(P, v.begin(), v.end(), 0); thrust::copy(P, ko.begin(), e.first, v.begin()); },
         { auto k = v; thrust::sort(k.begin(), k.end()); auto ko = v; auto vo = v;
           auto e = thrust::reduce_by_key(k.begin(), k.end(), v.begin(), ko.begin(), vo.begin(), thrust::equal_to<int>(), thrust::maximum<int>());
           thrust::fill(v.begin(), v.end(), 0); thrust::copy(ko.begin(), e.first, v.begin()); });
}
DECLARE_UNITTEST(TestReduceOverloads);

void TestTransformOverloads() {
  ON_ALL(thrust::for_each(P, v.begin(), v.end(), plus_one()), thrust::for_each(v.begin(), v.end(), plus_one()));
  ON_ALL(thrust::for_each_n(P, v.begin(), 10, plus_one()), thrust::for_each_n(v.begin(), 10, plus_one()));
  ON_ALL(thrust::transform(P, v.begin(), v.end(), v.begin(), twice()), thrust::transform(v.begin(), v.end(), v.begin(), twice()));
  ON_ALL(thrust::sequence(P, v.begin(), v.end(), 3, 2), thrust::sequence(v.begin(), v.end(), 3, 2));
  ON_ALL(thrust::fill(P, v.begin(), v.begin() + 10, 9), thrust::fill(v.begin(), v.begin() + 10, 9));
  ON_ALL(thrust::fill_n(P, v.begin(), 10, 9), thrust::fill_n(v.begin(), 10, 9));
  ON_ALL({ auto w = v; thrust::copy_n(P, w.begin() + 5, 20, v.begin()); }, { auto w = v; thrust::copy_n(w.begin() + 5, 20, v.begin()); });
  ON_ALL({ auto w = v; thrust::adjacent_difference(P, w.begin(), w.end(), v.begin()); }, { auto w = v; thrust::adjacent_difference(w.begin(), w.end(), v.begin()); });
  ON_ALL(thrust::adjacent_difference(P, v.begin(), v.end(), v.begin(), thrust::plus<int>()), thrust::adjacent_difference(v.begin(), v.end(), v.begin(), thrust::plus<int>()));
}
DECLARE_UNITTEST(TestTransformOverloads);

// compaction results: the tail beyond the new end is unspecified, so it is cleared before comparing
#define TRIM(V, END) thrust::fill((END), (V).end(), -1)
#define TRIMP(V, END) thrust::fill(P, (END), (V).end(), -1)
void TestSelectOverloads() {
  ON_ALL({ auto w = v; auto e = thrust::copy_if(P, w.begin(), w.end(), v.begin(), is_odd()); TRIMP(v, e); },
         { auto w = v; auto e = thrust::copy_if(w.begin(), w.end(), v.begin(), is_odd()); TRIM(v, e); });
  ON_ALL({ auto w = v; auto s = v; thrust::sequence(P, s.begin(), s.end()); auto e = thrust::copy_if(P, w.begin(), w.end(), s.begin(), v.begin(), is_odd()); TRIMP(v, e); },
         { auto w = v; auto s = v; thrust::sequence(s.begin(), s.end()); auto e = thrust::copy_if(w.begin(), w.end(), s.begin(), v.begin(), is_odd()); TRIM(v, e); });
  ON_ALL({ auto e = thrust::remove(P, v.begin(), v.end(), 3); TRIMP(v, e); }, { auto e = thrust::remove(v.begin(), v.end(), 3); TRIM(v, e); });
  ON_ALL({ auto e = thrust::remove_if(P, v.begin(), v.end(), is_odd()); TRIMP(v, e); }, { auto e = thrust::remove_if(v.begin(), v.end(), is_odd()); TRIM(v, e); });
  ON_ALL({ auto w = v; auto e = thrust::remove_copy(P, w.begin(), w.end(), v.begin(), 3); TRIMP(v, e); },
         { auto w = v; auto e = thrust::remove_copy_if(w.begin(), w.end(), v.begin(), thrust::detail::equals_value<int>{3}); TRIM(v, e); });
  ON_ALL({ thrust::sort(P, v.begin(), v.end()); auto e = thrust::unique(P, v.begin(), v.end()); TRIMP(v, e); },
         { thrust::sort(v.begin(), v.end()); auto e = thrust::unique(v.begin(), v.end()); TRIM(v, e); });
  ON_ALL({ thrust::sort(P, v.begin(), v.end()); auto e = thrust::unique(P, v.begin(), v.end(), same_half()); TRIMP(v, e); },
         { thrust::sort(v.begin(), v.end()); auto e = thrust::unique(v.begin(), v.end(), same_half()); TRIM(v, e); });
  ON_ALL({ thrust::sort(P, v.begin(), v.end()); auto w = v; auto e = thrust::unique_copy(P, w.begin(), w.end(), v.begin()); TRIMP(v, e); },
         { thrust::sort(v.begin(), v.end()); auto w = v; auto e = thrust::unique_copy(w.begin(), w.end(), v.begin()); TRIM(v, e); });
  ON_ALL({ thrust::sort(P, v.begin(), v.end()); auto w = v; auto e = thrust::unique_copy(P, w.begin(), w.end(), v.begin(), same_half()); TRIMP(v, e); },
         { thrust::sort(v.begin(), v.end()); auto w = v; auto e = thrust::unique_copy(w.begin(), w.end(), v.begin(), same_half()); TRIM(v, e); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); auto e = thrust::unique_by_key(P, k.begin(), k.end(), v.begin()); TRIMP(v, e.second); },
         { auto k = v; thrust::sort(k.begin(), k.end()); auto e = thrust::unique_by_key(k.begin(), k.end(), v.begin()); TRIM(v, e.second); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); auto e = thrust::unique_by_key(P, k.begin(), k.end(), v.begin(), same_half()); TRIMP(v, e.second); },
         { auto k = v; thrust::sort(k.begin(), k.end()); auto e = thrust::unique_by_key(k.begin(), k.end(), v.begin(), same_half()); TRIM(v, e.second); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); auto ko = v; auto w = v; auto e = thrust::unique_by_key_copy(P, k.begin(), k.end(), w.begin(), ko.begin(), v.begin()); TRIMP(v, e.second); },
         { auto k = v; thrust::sort(k.begin(), k.end()); auto ko = v; auto w = v; auto e = thrust::unique_by_key_copy(k.begin(), k.end(), w.begin(), ko.begin(), v.begin()); TRIM(v, e.second); });
  ON_ALL({ auto k = v; thrust::sort(P, k.begin(), k.end()); auto ko = v; auto w = v; auto e = thrust::unique_by_key_copy(P, k.begin(), k.end(), w.begin(), ko.begin(), v.begin(), same_half()); TRIMP(v, e.second); },
         { auto k = v; thrust::sort(k.begin(), k.end()); auto ko = v; auto w = v; auto e = thrust::unique_by_key_copy(k.begin(), k.end(), w.begin(), ko.begin(), v.begin(), same_half()); TRIM(v, e.second); });
}
DECLARE_UNITTEST(TestSelectOverloads);

void TestPartitionOverloads() {
  ON_ALL(thrust::partition(P, v.begin(), v.end(), is_odd()), thrust::partition(v.begin(), v.end(), is_odd()));
  ON_ALL(thrust::stable_partition(P, v.begin(), v.end(), is_odd()), thrust::stable_partition(v.begin(), v.end(), is_odd()));
  ON_ALL({ auto s = v; thrust::sequence(P, s.begin(), s.end()); thrust::partition(P, v.begin(), v.end(), s.begin(), is_odd()); },
         { auto s = v; thrust::sequence(s.begin(), s.end()); thrust::partition(v.begin(), v.end(), s.begin(), is_odd()); });
  ON_ALL({ auto s = v; thrust::sequence(P, s.begin(), s.end()); thrust::stable_partition(P, v.begin(), v.end(), s.begin(), is_odd()); },
         { auto s = v; thrust::sequence(s.begin(), s.end()); thrust::stable_partition(v.begin(), v.end(), s.begin(), is_odd()); });
  ON_ALL({ auto w = v; auto f = v; auto e = thrust::partition_copy(P, w.begin(), w.end(), v.begin(), f.begin(), is_odd()); thrust::copy(P, f.begin(), e.second, e.first); },
         { auto w = v; auto f = v; auto e = thrust::partition_copy(w.begin(), w.end(), v.begin(), f.begin(), is_odd()); thrust::copy(f.begin(), e.second, e.first); });
  ON_ALL({ auto w = v; auto f = v; auto s = v; thrust::sequence(P, s.begin(), s.end());
           auto e = thrust::stable_partition_copy(P, w.begin(), w.end(), s.begin(), v.begin(), f.begin(), is_odd()); thrust::copy(P, f.begin(), e.second, e.first); },
         { auto w = v; auto f = v; auto s = v; thrust::sequence(s.begin(), s.end());
           auto e = thrust::stable_partition_copy(w.begin(), w.end(), s.begin(), v.begin(), f.begin(), is_odd()); thrust::copy(f.begin(), e.second, e.first); });
}
DECLARE_UNITTEST(TestPartitionOverloads);

void TestSearchOverloads() {
  ON_ALL({ auto hay = v; thrust::sort(P, hay.begin(), hay.end()); auto q = v; thrust::lower_bound(P, hay.begin(), hay.end(), q.begin(), q.end(), v.begin()); },
         { auto hay = v; thrust::sort(hay.begin(), hay.end()); auto q = v; thrust::lower_bound(hay.begin(), hay.end(), q.begin(), q.end(), v.begin()); });
  ON_ALL({ auto hay = v; thrust::sort(P, hay.begin(), hay.end(), thrust::greater<int>()); auto q = v; thrust::upper_bound(P, hay.begin(), hay.end(), q.begin(), q.end(), v.begin(), thrust::greater<int>()); },
         { auto hay = v; thrust::sort(hay.begin(), hay.end(), thrust::greater<int>()); auto q = v; thrust::upper_bound(hay.begin(), hay.end(), q.begin(), q.end(), v.begin(), thrust::greater<int>()); });
  ON_ALL({ auto hay = v; thrust::sort(P, hay.begin(), hay.end()); auto q = v; thrust::sequence(P, q.begin(), q.end()); thrust::binary_search(P, hay.begin(), hay.end(), q.begin(), q.end(), v.begin()); },
         { auto hay = v; thrust::sort(hay.begin(), hay.end()); auto q = v; thrust::sequence(q.begin(), q.end()); thrust::binary_search(hay.begin(), hay.end(), q.begin(), q.end(), v.begin()); });
  ON_ALL({ thrust::sort(P, v.begin(), v.end()); const int a = (int)(thrust::lower_bound(P, v.begin(), v.end(), 25) - v.begin());
           const int b = (int)(thrust::upper_bound(P, v.begin(), v.end(), 25, thrust::less<int>()) - v.begin()); const bool c = thrust::binary_search(P, v.begin(), v.end(), 25);
           v[0] = a; v[1] = b; v[2] = c; },
         { thrust::sort(v.begin(), v.end()); const int a = (int)(thrust::lower_bound(v.begin(), v.end(), 25) - v.begin());
           const int b = (int)(thrust::upper_bound(v.begin(), v.end(), 25) - v.begin()); const bool c = thrust::binary_search(v.begin(), v.end(), 25);
           v[0] = a; v[1] = b; v[2] = c; });
}
DECLARE_UNITTEST(TestSearchOverloads);

// the rest of the vector's container interface (thrust/detail/vector_base.h:240-470)
void TestDeviceVectorReverseIterationAndCheckedAccess() {
  thrust::device_vector<int> v(5);
  for (int i = 0; i < 5; i++) v[i] = i * i;
  ASSERT_EQUAL((int)v.at(3), 9);
  ASSERT_THROWS(v.at(5), std::out_of_range);
  ASSERT_EQUAL((int)*v.rbegin(), 16);
  ASSERT_EQUAL((int)(v.rend() - v.rbegin()), 5);
  thrust::host_vector<int> back(v.rbegin(), v.rend());
  ASSERT_EQUAL(back[0], 16);
  ASSERT_EQUAL(back[4], 0);
  const thrust::device_vector<int>& c = v;
  ASSERT_EQUAL((int)*c.crbegin(), 16);
  ASSERT_EQUAL((int)c.at(1), 1);
  ASSERT_TRUE(v.max_size() >= v.size());
  static_assert(std::is_same<thrust::device_vector<int>::difference_type, std::ptrdiff_t>::value, "");
}
DECLARE_UNITTEST(TestDeviceVectorReverseIterationAndCheckedAccess);

// ---- vectors convert between systems, element types and allocators (thrust/detail/vector_base.h:153-185)
void TestVectorConversions() {
  thrust::host_vector<int> hi(100);
  for (int i = 0; i < 100; i++) hi[i] = i - 50;
  thrust::device_vector<float> df(hi);            // host int -> device float
  thrust::device_vector<double> dd(df);           // device float -> device double
  thrust::host_vector<long> hl(dd);               // device double -> host long
  for (int i = 0; i < 100; i++) ASSERT_EQUAL(hl[i], (long)(i - 50));
  std::vector<short> sv{1, 2, 3};
  thrust::device_vector<int> ds(sv);
  ASSERT_EQUAL(ds == (thrust::host_vector<int>{1, 2, 3}), true);
  ASSERT_EQUAL(ds == (std::vector<long>{1, 2, 3}), true);
  ASSERT_EQUAL((thrust::host_vector<int>{1, 2, 4}) != ds, true);
  ds = hi;                                        // assignment across systems
  ASSERT_EQUAL(ds.size(), std::size_t(100));
  ASSERT_EQUAL((int)ds[99], 49);
  df = ds;                                        // and across element types
  ASSERT_EQUAL((float)df[0], -50.0f);
  thrust::host_vector<bool> hb(9, false);
  hb[4] = true;
  thrust::device_vector<bool> db = hb;            // bool elements are bytes on both sides
  thrust::host_vector<bool> back = db;
  ASSERT_EQUAL(back == hb, true);
  ASSERT_EQUAL((bool)db[4], true);
  thrust::host_vector<int> from_fancy(thrust::make_transform_iterator(ds.begin(), thrust::negate<int>()),
                                      thrust::make_transform_iterator(ds.end(), thrust::negate<int>()));
  ASSERT_EQUAL(from_fancy[0], 50);
  thrust::host_vector<int> from_counting(thrust::counting_iterator<int>(3), thrust::counting_iterator<int>(6));
  ASSERT_EQUAL(from_counting == (std::vector<int>{3, 4, 5}), true);
  ds.insert(ds.begin() + 1, 3, 7);
  ASSERT_EQUAL((int)ds[1], 7); ASSERT_EQUAL((int)ds[3], 7); ASSERT_EQUAL((int)ds[4], -49);
  ASSERT_EQUAL(ds.size(), std::size_t(103));
  // move assignment hands the storage over and leaves the source empty (testing/vector.cu:814-826)
  thrust::device_vector<int> m1(3, 1), m2(2, 2);
  const int* held = thrust::raw_pointer_cast(m1.data());
  m2 = std::move(m1);
  ASSERT_EQUAL(m1.empty(), true);
  ASSERT_EQUAL(m2.size(), std::size_t(3));
  ASSERT_EQUAL(thrust::raw_pointer_cast(m2.data()) == held, true);
  ASSERT_EQUAL((int)m2[2], 1);
}
DECLARE_UNITTEST(TestVectorConversions);

// ---- thrust::copy between every pair of systems and iterator kinds, without a policy
void TestCopyBetweenEveryPairOfSystems() {
  const int n = 1000;
  thrust::host_vector<int> h(n);
  for (int i = 0; i < n; i++) h[i] = 3 * i;
  thrust::device_vector<int> d(n), d2(n);
  thrust::copy(h.begin(), h.end(), d.begin());                          // host -> device
  thrust::copy(d.begin(), d.end(), d2.begin());                         // device -> device
  thrust::device_vector<float> df(n);
  thrust::copy(d.begin(), d.end(), df.begin());                         // device -> device, converting
  ASSERT_EQUAL((float)df[n - 1], 3.0f * (n - 1));
  thrust::host_vector<int> back(n);
  thrust::copy(d2.begin(), d2.end(), back.begin());                     // device -> host
  ASSERT_EQUAL(back, h);
  thrust::device_vector<int> da(n), db(n);
  thrust::host_vector<thrust::tuple<int, int>> aos(n);
  for (int i = 0; i < n; i++) aos[i] = thrust::make_tuple(i, -i);
  thrust::copy(aos.begin(), aos.end(), thrust::make_zip_iterator(thrust::make_tuple(da.begin(), db.begin())));  // host -> zipped device
  ASSERT_EQUAL((int)da[7], 7); ASSERT_EQUAL((int)db[7], -7);
  thrust::device_vector<int> dc(n), dd(n);
  thrust::copy(thrust::make_zip_iterator(thrust::make_tuple(da.begin(), db.begin())),
               thrust::make_zip_iterator(thrust::make_tuple(da.end(), db.end())),
               thrust::make_zip_iterator(thrust::make_tuple(dc.begin(), dd.begin())));                          // zipped device -> zipped device
  ASSERT_EQUAL(dc, da); ASSERT_EQUAL(dd, db);
  auto e1 = thrust::copy(h.begin(), h.end(), thrust::make_discard_iterator());                                  // host -> nowhere
  auto e2 = thrust::copy(d.begin(), d.end(), thrust::make_discard_iterator());                                  // device -> nowhere
  ASSERT_EQUAL((int)(e1 - thrust::make_discard_iterator()), n);
  ASSERT_EQUAL((int)(e2 - thrust::make_discard_iterator()), n);
  thrust::host_vector<int> hc(5);
  thrust::copy(thrust::counting_iterator<int>(10), thrust::counting_iterator<int>(15), hc.begin());             // counting -> host, on the host
  ASSERT_EQUAL(hc[4], 14);
  thrust::copy_n(thrust::counting_iterator<int>(10), 5, d.begin());                                             // counting -> device
  ASSERT_EQUAL((int)d[4], 14);
  std::list<int> l{5, 6, 7};
  thrust::copy_n(l.begin(), 3, d.begin());                                                                      // a stepping host iterator
  ASSERT_EQUAL((int)d[2], 7);
}
DECLARE_UNITTEST(TestCopyBetweenEveryPairOfSystems);

// ---- device_reference behaves like the element (thrust/device_reference.h:224-970)
void TestDeviceReferenceArithmetic() {
  thrust::device_vector<int> v(2, 10);
  thrust::device_reference<int> r = v[0];
  r += 5; ASSERT_EQUAL((int)v[0], 15);
  r -= 1; r *= 2; ASSERT_EQUAL((int)v[0], 28);
  r /= 7; r %= 3; ASSERT_EQUAL((int)v[0], 1);
  r <<= 4; r |= 1; r ^= 3; r &= 0xfe; r >>= 1; ASSERT_EQUAL((int)v[0], 9);
  ++r; ASSERT_EQUAL((int)r, 10);
  ASSERT_EQUAL(r++, 10); ASSERT_EQUAL((int)r, 11);
  --r; r--; ASSERT_EQUAL((int)v[0], 9);
  thrust::device_reference<int> q(v.data() + 1);
  q = r;
  ASSERT_EQUAL((int)v[1], 9);
  v[1] = 4;
  thrust::swap(r, q);
  ASSERT_EQUAL((int)v[0], 4); ASSERT_EQUAL((int)v[1], 9);
  thrust::device_reference<const int> c = v[1];
  ASSERT_EQUAL((int)c, 9);
  std::ostringstream os;
  os << r << ' ' << (v.data() != thrust::device_ptr<int>());
  ASSERT_EQUAL(os.str() == std::string("4 1"), true);
}
DECLARE_UNITTEST(TestDeviceReferenceArithmetic);

// ---- thrust::pointer carries its system; universal_vector is a class of its own
struct tagged_policy : thrust::device_execution_policy<tagged_policy> {};
template <class T> int which_vector(const thrust::device_vector<T>&) { return 1; }
template <class T> int which_vector(const thrust::universal_vector<T>&) { return 2; }
void TestTaggedPointerAndUniversalVector() {
  thrust::device_vector<int> v(100);
  thrust::pointer<int, thrust::device_system_tag> p(thrust::raw_pointer_cast(v.data()));
  thrust::sequence(p, p + 100);
  ASSERT_EQUAL(thrust::reduce(p, p + 100), 4950);
  ASSERT_EQUAL((int)p[7], 7);
  *p = 3;
  ASSERT_EQUAL((int)v[0], 3);
  thrust::pointer<int, tagged_policy> t(thrust::raw_pointer_cast(v.data()));
  thrust::fill(t, t + 100, 2);  // runs on the device under the user's (overload-free) policy type
  ASSERT_EQUAL(thrust::reduce(v.begin(), v.end()), 200);
  int host_array[4] = {4, 3, 2, 1};
  thrust::pointer<int, thrust::host_system_tag> hp(host_array);
  thrust::sort(hp, hp + 4);
  ASSERT_EQUAL(host_array[0], 1); ASSERT_EQUAL(*hp, 1);
  thrust::universal_vector<int> u(10, 1);
  thrust::device_vector<int> d(10, 1);
  ASSERT_EQUAL(which_vector(u), 2);
  ASSERT_EQUAL(which_vector(d), 1);
  ASSERT_EQUAL(thrust::reduce(u.begin(), u.end()), 10);
  u = d;
  thrust::universal_vector<int> u2 = u;
  ASSERT_EQUAL(u2.size(), std::size_t(10));
}
DECLARE_UNITTEST(TestTaggedPointerAndUniversalVector);

// ---- a number-like struct with written-out copy operations as an element
// (custom_numeric of testing/unittest/testframework.h:128-232)
struct numberlike {
  int v[2];
  __host__ __device__ numberlike() { v[0] = v[1] = 0; }
  __host__ __device__ numberlike(int x) { v[0] = v[1] = x; }
  __host__ __device__ numberlike(const numberlike& o) { v[0] = o.v[0]; v[1] = o.v[1]; }
  __host__ __device__ numberlike& operator=(const numberlike& o) { v[0] = o.v[0]; v[1] = o.v[1]; return *this; }
  __host__ __device__ numberlike operator+(const numberlike& o) const { return numberlike(v[0] + o.v[0]); }
  __host__ __device__ numberlike operator*(const numberlike& o) const { return numberlike(v[0] * o.v[0]); }
  __host__ __device__ bool operator<(const numberlike& o) const { return v[0] < o.v[0]; }
  __host__ __device__ bool operator==(const numberlike& o) const { return v[0] == o.v[0] && v[1] == o.v[1]; }
};
inline std::ostream& operator<<(std::ostream& os, const numberlike& x) { return os << x.v[0]; }
void TestNumberLikeStructElements() {
  const int n = 5000;
  thrust::host_vector<numberlike> h(n);
  for (int i = 0; i < n; i++) h[i] = numberlike((i * 7919) % 1000);
  thrust::device_vector<numberlike> d = h, out(n);
  ASSERT_EQUAL(thrust::reduce(d.begin(), d.end(), numberlike(0), thrust::plus<numberlike>()) ==
                   std::accumulate(h.begin(), h.end(), numberlike(0), thrust::plus<numberlike>()), true);
  thrust::inclusive_scan(d.begin(), d.end(), out.begin(), thrust::plus<numberlike>());
  thrust::host_vector<numberlike> hs(n);
  std::partial_sum(h.begin(), h.end(), hs.begin(), thrust::plus<numberlike>());
  ASSERT_EQUAL(out == hs, true);
  thrust::sort(d.begin(), d.end());
  std::stable_sort(h.begin(), h.end());
  ASSERT_EQUAL(d == h, true);
  thrust::device_vector<numberlike> seq(8);
  thrust::sequence(seq.begin(), seq.end(), numberlike(1), numberlike(2));
  ASSERT_EQUAL(((numberlike)seq[3]).v[0], 7);
}
DECLARE_UNITTEST(TestNumberLikeStructElements);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
