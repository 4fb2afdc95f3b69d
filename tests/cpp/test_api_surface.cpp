// Every public overload once: with thrust::device, with a stream policy, with thrust::host and
// without a policy on device and host ranges.  Mostly a compile check of the overload sets
// (templates that no other test instantiates); each call's result is also compared between the
// host and the device range.  Compiled by hipcc.
#include <thrust/adjacent_difference.h>
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

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
