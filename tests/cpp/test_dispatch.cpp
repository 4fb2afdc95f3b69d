// Customisation by policy type: an algorithm called with a policy derived from
// thrust::device_execution_policy<my_system> — or WITHOUT a policy on iterators retagged with such
// a type — reaches the user's overload for that type, and the device system's implementation when
// there is none.  After the Test*DispatchExplicit / Test*DispatchImplicit pairs of testing/sort.cu:8-40,
// testing/stable_sort.cu, sort_by_key.cu, stable_sort_by_key.cu, scan.cu:19-90, scan_by_key.inclusive.cu,
// scan_by_key.exclusive.cu, reduce_by_key.cu and reduce.cu, with my_system / my_tag of
// testing/unittest/special_types.h:135-170.  Compiled by hipcc (retagged iterators are fancy iterators: kernel templates).
#include <thrust/copy.h>
#include <thrust/execution_policy.h>
#include <thrust/fill.h>
#include <thrust/iterator/retag.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sort.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>

#include "testing.h"

// counts its copies: dispatch must hand the caller's own object to the overload
class my_system : public thrust::device_execution_policy<my_system> {
 public:
  explicit my_system(int) : correctly_dispatched(false), num_copies(0) {}
  my_system(const my_system& other) : thrust::device_execution_policy<my_system>(other), correctly_dispatched(false), num_copies(other.num_copies + 1) {}
  void validate_dispatch() { correctly_dispatched = (num_copies == 0); }
  bool is_valid() const { return correctly_dispatched; }

 private:
  bool correctly_dispatched;
  unsigned int num_copies;
};
struct my_tag : thrust::device_execution_policy<my_tag> {};

// ---- the user's overloads ------------------------------------------------------------------
template <class It> void sort(my_system& s, It, It) { s.validate_dispatch(); }
template <class It> void sort(my_tag, It first, It) { *first = 13; }
template <class It> void stable_sort(my_system& s, It, It) { s.validate_dispatch(); }
template <class It> void stable_sort(my_tag, It first, It) { *first = 13; }
template <class K, class V> void sort_by_key(my_system& s, K, K, V) { s.validate_dispatch(); }
template <class K, class V> void sort_by_key(my_tag, K first, K, V) { *first = 13; }
template <class K, class V> void stable_sort_by_key(my_system& s, K, K, V) { s.validate_dispatch(); }
template <class K, class V> void stable_sort_by_key(my_tag, K first, K, V) { *first = 13; }
template <class In, class Out> Out inclusive_scan(my_system& s, In, In, Out r) { s.validate_dispatch(); return r; }
template <class In, class Out> Out inclusive_scan(my_tag, In, In, Out r) { *r = 13; return r; }
template <class In, class Out> Out exclusive_scan(my_system& s, In, In, Out r) { s.validate_dispatch(); return r; }
template <class In, class Out> Out exclusive_scan(my_tag, In, In, Out r) { *r = 13; return r; }
template <class K, class V, class Out> Out inclusive_scan_by_key(my_system& s, K, K, V, Out r) { s.validate_dispatch(); return r; }
template <class K, class V, class Out> Out inclusive_scan_by_key(my_tag, K, K, V, Out r) { *r = 13; return r; }
template <class K, class V, class Out> Out exclusive_scan_by_key(my_system& s, K, K, V, Out r) { s.validate_dispatch(); return r; }
template <class K, class V, class Out> Out exclusive_scan_by_key(my_tag, K, K, V, Out r) { *r = 13; return r; }
template <class K, class V, class KO, class VO>
thrust::pair<KO, VO> reduce_by_key(my_system& s, K, K, V, KO ko, VO vo) { s.validate_dispatch(); return thrust::make_pair(ko, vo); }
template <class K, class V, class KO, class VO>
thrust::pair<KO, VO> reduce_by_key(my_tag, K, K, V, KO ko, VO vo) { *ko = 13; return thrust::make_pair(ko, vo); }
template <class It> int reduce(my_system& s, It, It) { s.validate_dispatch(); return 13; }
template <class It> int reduce(my_tag, It, It) { return 13; }

template <class In, class Out> Out copy(my_system& s, In, In, Out r) { s.validate_dispatch(); return r; }
template <class In, class Out> Out copy(my_tag, In, In, Out r) { *r = 13; return r; }
template <class In, class Out, class P> Out copy_if(my_system& s, In, In, Out r, P) { s.validate_dispatch(); return r; }
template <class In, class Out, class P> Out copy_if(my_system& s, In, In, In, Out r, P) { s.validate_dispatch(); return r; }
template <class It, class T> void fill(my_system& s, It, It, const T&) { s.validate_dispatch(); }
template <class In, class Out, class F> Out transform(my_system& s, In, In, Out r, F) { s.validate_dispatch(); return r; }
template <class In, class Out, class F> Out transform(my_system& s, In, In, In, Out r, F) { s.validate_dispatch(); return r; }
template <class In, class F, class T, class Op> T transform_reduce(my_system& s, In, In, F, T init, Op) { s.validate_dispatch(); return init; }

#define EXPLICIT(NAME, ...)                    \
  void Test_##NAME##_DispatchExplicit() {      \
    thrust::device_vector<int> vec(1);         \
    my_system sys(0);                          \
    thrust::NAME(sys, __VA_ARGS__);            \
    ASSERT_EQUAL(true, sys.is_valid());        \
  }                                            \
  DECLARE_UNITTEST(Test_##NAME##_DispatchExplicit)
#define IMPLICIT(NAME, ...)                    \
  void Test_##NAME##_DispatchImplicit() {      \
    thrust::device_vector<int> vec(1);         \
    thrust::NAME(__VA_ARGS__);                 \
    ASSERT_EQUAL(13, (int)vec.front());        \
  }                                            \
  DECLARE_UNITTEST(Test_##NAME##_DispatchImplicit)
#define B vec.begin()
#define T thrust::retag<my_tag>(vec.begin())

EXPLICIT(sort, B, B);
IMPLICIT(sort, T, T);
EXPLICIT(stable_sort, B, B);
IMPLICIT(stable_sort, T, T);
EXPLICIT(sort_by_key, B, B, B);
IMPLICIT(sort_by_key, T, T, T);
EXPLICIT(stable_sort_by_key, B, B, B);
IMPLICIT(stable_sort_by_key, T, T, T);
EXPLICIT(inclusive_scan, B, B, B);
IMPLICIT(inclusive_scan, T, T, T);
EXPLICIT(exclusive_scan, B, B, B);
IMPLICIT(exclusive_scan, T, T, T);
EXPLICIT(inclusive_scan_by_key, B, B, B, B);
IMPLICIT(inclusive_scan_by_key, T, T, T, T);
EXPLICIT(exclusive_scan_by_key, B, B, B, B);
IMPLICIT(exclusive_scan_by_key, T, T, T, T);
EXPLICIT(reduce_by_key, B, B, B, B, B);
IMPLICIT(reduce_by_key, T, T, T, T, T);
EXPLICIT(reduce, B, B);

EXPLICIT(copy, B, B, B);
IMPLICIT(copy, T, T, T);
EXPLICIT(copy_if, B, B, B, thrust::identity<int>());
void TestCopyIfStencilDispatchExplicit() {
  thrust::device_vector<int> vec(1);
  my_system sys(0);
  thrust::copy_if(sys, B, B, B, B, thrust::identity<int>());
  ASSERT_EQUAL(true, sys.is_valid());
}
DECLARE_UNITTEST(TestCopyIfStencilDispatchExplicit);
EXPLICIT(fill, B, B, 0);
EXPLICIT(transform, B, B, B, thrust::negate<int>());
void TestBinaryTransformDispatchExplicit() {
  thrust::device_vector<int> vec(1);
  my_system sys(0);
  thrust::transform(sys, B, B, B, B, thrust::plus<int>());
  ASSERT_EQUAL(true, sys.is_valid());
}
DECLARE_UNITTEST(TestBinaryTransformDispatchExplicit);
EXPLICIT(transform_reduce, B, B, thrust::negate<int>(), 0, thrust::plus<int>());

void TestReduceDispatchImplicit() {
  thrust::device_vector<int> vec(1);
  ASSERT_EQUAL(13, thrust::reduce(thrust::retag<my_tag>(vec.begin()), thrust::retag<my_tag>(vec.begin())));
}
DECLARE_UNITTEST(TestReduceDispatchImplicit);

// sort reaches a user's stable_sort, as the generic layer's sort does (thrust/system/detail/generic/sort.inl:56-62)
struct only_stable : thrust::device_execution_policy<only_stable> { bool hit = false; };
template <class It> void stable_sort(only_stable& s, It, It) { s.hit = true; }
template <class K, class V> void stable_sort_by_key(only_stable& s, K, K, V) { s.hit = true; }
void TestSortFallsToTheUsersStableSort() {
  thrust::device_vector<int> vec(3);
  only_stable a, b;
  thrust::sort(a, vec.begin(), vec.end());
  ASSERT_TRUE(a.hit);
  thrust::sort_by_key(b, vec.begin(), vec.end(), vec.begin());
  ASSERT_TRUE(b.hit);
}
DECLARE_UNITTEST(TestSortFallsToTheUsersStableSort);

// a policy type without overloads of its own, and retagged iterators without a user policy, run the
// device system's implementation
struct plain_policy : thrust::device_execution_policy<plain_policy> {};
void TestPolicyWithoutOverloadsRunsTheDeviceSystem() {
  const int n = 10000;
  thrust::host_vector<int> h(n);
  for (int i = 0; i < n; i++) h[i] = (i * 7919) % 1000;
  thrust::device_vector<int> d = h, out(n), keys(n, 1), ko(n), vo(n);
  plain_policy p;
  thrust::sort(p, d.begin(), d.end());
  std::sort(h.begin(), h.end());
  ASSERT_EQUAL(thrust::host_vector<int>(d), h);
  thrust::inclusive_scan(p, d.begin(), d.end(), out.begin());
  long long sum = 0;
  for (int i = 0; i < n; i++) sum += h[i];
  ASSERT_EQUAL((long long)(int)out.back(), sum);
  ASSERT_EQUAL((long long)thrust::reduce(p, d.begin(), d.end()), sum);
  auto ends = thrust::reduce_by_key(p, keys.begin(), keys.end(), d.begin(), ko.begin(), vo.begin());
  ASSERT_EQUAL((int)(ends.first - ko.begin()), 1);
  ASSERT_EQUAL((long long)(int)vo[0], sum);
  thrust::exclusive_scan_by_key(p, keys.begin(), keys.end(), d.begin(), out.begin());
  ASSERT_EQUAL((int)out[0], 0);
  ASSERT_EQUAL((long long)(int)out.back(), sum - h[n - 1]);
  // retag to the device system's own tag: the no-policy forms run on the device
  thrust::device_vector<int> e = thrust::host_vector<int>(h.rbegin(), h.rend());
  thrust::sort(thrust::retag<thrust::device_system_tag>(e.begin()), thrust::retag<thrust::device_system_tag>(e.end()));
  ASSERT_EQUAL(thrust::host_vector<int>(e), h);
}
DECLARE_UNITTEST(TestPolicyWithoutOverloadsRunsTheDeviceSystem);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
