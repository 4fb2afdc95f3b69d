// Customisation by policy type: an algorithm called with a policy derived from
// thrust::device_execution_policy<my_system> — or WITHOUT a policy on iterators retagged with such
// a type — reaches the user's overload for that type, and the device system's implementation when
// there is none.  After the Test*DispatchExplicit / Test*DispatchImplicit pairs of testing/sort.cu:8-40,
// testing/stable_sort.cu, sort_by_key.cu, stable_sort_by_key.cu, scan.cu:19-90, scan_by_key.inclusive.cu,
// scan_by_key.exclusive.cu, reduce_by_key.cu and reduce.cu, with my_system / my_tag of
// testing/unittest/special_types.h:135-170.  Compiled by hipcc (retagged iterators are fancy iterators: kernel templates).
#include <thrust/adjacent_difference.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/equal.h>
#include <thrust/for_each.h>
#include <thrust/transform_scan.h>
#include <thrust/logical.h>
#include <thrust/extrema.h>
#include <thrust/find.h>
#include <thrust/gather.h>
#include <thrust/generate.h>
#include <thrust/inner_product.h>
#include <thrust/merge.h>
#include <thrust/mismatch.h>
#include <thrust/partition.h>
#include <thrust/random.h>
#include <thrust/remove.h>
#include <thrust/replace.h>
#include <thrust/reverse.h>
#include <thrust/scatter.h>
#include <thrust/sequence.h>
#include <thrust/shuffle.h>
#include <thrust/swap.h>
#include <thrust/tabulate.h>
#include <thrust/uninitialized_copy.h>
#include <thrust/uninitialized_fill.h>
#include <thrust/unique.h>
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
#define BEGIN_ vec.begin()
#define TAGGED_ thrust::retag<my_tag>(vec.begin())

EXPLICIT(sort, BEGIN_, BEGIN_);
IMPLICIT(sort, TAGGED_, TAGGED_);
EXPLICIT(stable_sort, BEGIN_, BEGIN_);
IMPLICIT(stable_sort, TAGGED_, TAGGED_);
EXPLICIT(sort_by_key, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(sort_by_key, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(stable_sort_by_key, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(stable_sort_by_key, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(inclusive_scan, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(inclusive_scan, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(exclusive_scan, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(exclusive_scan, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(inclusive_scan_by_key, BEGIN_, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(inclusive_scan_by_key, TAGGED_, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(exclusive_scan_by_key, BEGIN_, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(exclusive_scan_by_key, TAGGED_, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(reduce_by_key, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(reduce_by_key, TAGGED_, TAGGED_, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(reduce, BEGIN_, BEGIN_);

EXPLICIT(copy, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(copy, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(copy_if, BEGIN_, BEGIN_, BEGIN_, thrust::identity<int>());
void TestCopyIfStencilDispatchExplicit() {
  thrust::device_vector<int> vec(1);
  my_system sys(0);
  thrust::copy_if(sys, BEGIN_, BEGIN_, BEGIN_, BEGIN_, thrust::identity<int>());
  ASSERT_EQUAL(true, sys.is_valid());
}
DECLARE_UNITTEST(TestCopyIfStencilDispatchExplicit);
EXPLICIT(fill, BEGIN_, BEGIN_, 0);
EXPLICIT(transform, BEGIN_, BEGIN_, BEGIN_, thrust::negate<int>());
void TestBinaryTransformDispatchExplicit() {
  thrust::device_vector<int> vec(1);
  my_system sys(0);
  thrust::transform(sys, BEGIN_, BEGIN_, BEGIN_, BEGIN_, thrust::plus<int>());
  ASSERT_EQUAL(true, sys.is_valid());
}
DECLARE_UNITTEST(TestBinaryTransformDispatchExplicit);
EXPLICIT(transform_reduce, BEGIN_, BEGIN_, thrust::negate<int>(), 0, thrust::plus<int>());


// ---- the other algorithms: the form that names every operator dispatches on the policy type (the
//      shorter forms supply the default operator and call it) --------------------------------
#define V(x) s.validate_dispatch(); return x
template <class In, class Out, class Op> Out adjacent_difference(my_system& s, In, In, Out r, Op) { V(r); }
template <class It, class C> It min_element(my_system& s, It f, It, C) { V(f); }
template <class It, class C> It max_element(my_system& s, It f, It, C) { V(f); }
template <class It, class C> thrust::pair<It, It> minmax_element(my_system& s, It f, It, C) { V(thrust::make_pair(f, f)); }
template <class It, class P> It find_if(my_system& s, It f, It, P) { V(f); }
template <class It, class P> It find_if_not(my_system& s, It f, It, P) { V(f); }
template <class M, class In, class Out> Out gather(my_system& s, M, M, In, Out r) { V(r); }
template <class M, class S, class In, class Out, class P> Out gather_if(my_system& s, M, M, S, In, Out r, P) { V(r); }
template <class It, class G> void generate(my_system& s, It, It, G) { s.validate_dispatch(); }
template <class A, class Bi, class T, class O1, class O2> T inner_product(my_system& s, A, A, Bi, T init, O1, O2) { V(init); }
template <class A, class Bi, class Out, class C> Out merge(my_system& s, A, A, Bi, Bi, Out r, C) { V(r); }
template <class A, class Bi, class VA, class VBB, class KO, class VO, class C>
thrust::pair<KO, VO> merge_by_key(my_system& s, A, A, Bi, Bi, VA, VBB, KO ko, VO vo, C) { V(thrust::make_pair(ko, vo)); }
template <class A, class Bi, class P> thrust::pair<A, Bi> mismatch(my_system& s, A a, A, Bi b, P) { V(thrust::make_pair(a, b)); }
template <class It, class P> It stable_partition(my_system& s, It f, It, P) { V(f); }
template <class In, class O1, class O2, class P> thrust::pair<O1, O2> stable_partition_copy(my_system& s, In, In, O1 a, O2 b, P) { V(thrust::make_pair(a, b)); }
template <class In, class Out, class P> Out remove_copy_if(my_system& s, In, In, Out r, P) { V(r); }
template <class It, class P> It remove_if(my_system& s, It f, It, P) { V(f); }
template <class In, class S, class Out, class P, class T> Out replace_copy_if(my_system& s, In, In, S, Out r, P, const T&) { V(r); }
template <class It> void reverse(my_system& s, It, It) { s.validate_dispatch(); }
template <class In, class Out> Out reverse_copy(my_system& s, In, In, Out r) { V(r); }
template <class In, class M, class Out> void scatter(my_system& s, In, In, M, Out) { s.validate_dispatch(); }
template <class In, class M, class S, class Out, class P> void scatter_if(my_system& s, In, In, M, S, Out, P) { s.validate_dispatch(); }
template <class It, class T> void sequence(my_system& s, It, It, T, T) { s.validate_dispatch(); }
template <class It, class G> void shuffle(my_system& s, It, It, G&&) { s.validate_dispatch(); }
template <class In, class Out, class G> void shuffle_copy(my_system& s, In, In, Out, G&&) { s.validate_dispatch(); }
template <class A, class Bi> Bi swap_ranges(my_system& s, A, A, Bi b) { V(b); }
template <class It, class F> void tabulate(my_system& s, It, It, F) { s.validate_dispatch(); }
template <class In, class Out> Out uninitialized_copy(my_system& s, In, In, Out r) { V(r); }
template <class It, class T> void uninitialized_fill(my_system& s, It, It, const T&) { s.validate_dispatch(); }
template <class It, class E> It unique(my_system& s, It f, It, E) { V(f); }
template <class In, class Out, class E> Out unique_copy(my_system& s, In, In, Out r, E) { V(r); }
template <class K, class Vi, class E> thrust::pair<K, Vi> unique_by_key(my_system& s, K k, K, Vi v, E) { V(thrust::make_pair(k, v)); }
template <class K, class Vi, class KO, class VO, class E>
thrust::pair<KO, VO> unique_by_key_copy(my_system& s, K, K, Vi, KO ko, VO vo, E) { V(thrust::make_pair(ko, vo)); }
#undef V

typedef thrust::less<int> L;
typedef thrust::equal_to<int> E;
typedef thrust::identity<int> I;
EXPLICIT(adjacent_difference, BEGIN_, BEGIN_, BEGIN_, thrust::minus<int>());
EXPLICIT(min_element, BEGIN_, BEGIN_, L());
EXPLICIT(max_element, BEGIN_, BEGIN_, L());
EXPLICIT(minmax_element, BEGIN_, BEGIN_, L());
EXPLICIT(find_if, BEGIN_, BEGIN_, I());
EXPLICIT(find_if_not, BEGIN_, BEGIN_, I());
EXPLICIT(gather, BEGIN_, BEGIN_, BEGIN_, BEGIN_);
EXPLICIT(gather_if, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, I());
EXPLICIT(generate, BEGIN_, BEGIN_, thrust::default_random_engine());
EXPLICIT(inner_product, BEGIN_, BEGIN_, BEGIN_, 0, thrust::plus<int>(), thrust::multiplies<int>());
EXPLICIT(merge, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, L());
EXPLICIT(merge_by_key, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, L());
EXPLICIT(mismatch, BEGIN_, BEGIN_, BEGIN_, E());
EXPLICIT(stable_partition, BEGIN_, BEGIN_, I());
EXPLICIT(stable_partition_copy, BEGIN_, BEGIN_, BEGIN_, BEGIN_, I());
EXPLICIT(remove_copy_if, BEGIN_, BEGIN_, BEGIN_, I());
EXPLICIT(remove_if, BEGIN_, BEGIN_, I());
EXPLICIT(replace_copy_if, BEGIN_, BEGIN_, BEGIN_, BEGIN_, I(), 0);
EXPLICIT(reverse, BEGIN_, BEGIN_);
EXPLICIT(reverse_copy, BEGIN_, BEGIN_, BEGIN_);
EXPLICIT(scatter, BEGIN_, BEGIN_, BEGIN_, BEGIN_);
EXPLICIT(scatter_if, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, I());
EXPLICIT(sequence, BEGIN_, BEGIN_, 0, 1);
EXPLICIT(shuffle, BEGIN_, BEGIN_, thrust::default_random_engine());
EXPLICIT(shuffle_copy, BEGIN_, BEGIN_, BEGIN_, thrust::default_random_engine());
EXPLICIT(swap_ranges, BEGIN_, BEGIN_, BEGIN_);
EXPLICIT(tabulate, BEGIN_, BEGIN_, I());
EXPLICIT(uninitialized_copy, BEGIN_, BEGIN_, BEGIN_);
EXPLICIT(uninitialized_fill, BEGIN_, BEGIN_, 0);
EXPLICIT(unique, BEGIN_, BEGIN_, E());
EXPLICIT(unique_copy, BEGIN_, BEGIN_, BEGIN_, E());
EXPLICIT(unique_by_key, BEGIN_, BEGIN_, BEGIN_, E());
EXPLICIT(unique_by_key_copy, BEGIN_, BEGIN_, BEGIN_, BEGIN_, BEGIN_, E());

// ---- algorithms composed from others dispatch on the policy's own type too, and every form
//      without a policy takes the policy of retagged iterators (testing/{partition_point,
//      is_partitioned,logical,generate,replace,transform,transform_scan,remove,for_each,equal,find}.cu)
#define V(x) s.validate_dispatch(); return x
template <class It, class P> It partition_point(my_system& s, It f, It, P) { V(f); }
template <class It, class P> It partition_point(my_tag, It f, It, P) { *f = 13; return f; }
template <class It, class P> bool is_partitioned(my_system& s, It, It, P) { V(false); }
template <class It, class P> bool is_partitioned(my_tag, It f, It, P) { *f = 13; return false; }
template <class It, class P> bool all_of(my_system& s, It, It, P) { V(false); }
template <class It, class P> bool all_of(my_tag, It f, It, P) { *f = 13; return false; }
template <class It, class P> bool any_of(my_system& s, It, It, P) { V(false); }
template <class It, class P> bool none_of(my_system& s, It, It, P) { V(false); }
template <class It, class N, class G> It generate_n(my_system& s, It f, N, G) { V(f); }
template <class It, class N, class G> It generate_n(my_tag, It f, N, G) { *f = 13; return f; }
template <class It, class G> void generate(my_tag, It f, It, G) { *f = 13; }
template <class It, class P, class T> void replace_if(my_system& s, It, It, P, const T&) { s.validate_dispatch(); }
template <class It, class P, class T> void replace_if(my_tag, It f, It, P, const T&) { *f = 13; }
template <class It, class T> void replace(my_system& s, It, It, const T&, const T&) { s.validate_dispatch(); }
template <class In, class Out, class F, class P> Out transform_if(my_system& s, In, In, Out r, F, P) { V(r); }
template <class In, class Out, class F, class P> Out transform_if(my_tag, In, In, Out r, F, P) { *r = 13; return r; }
template <class In, class St, class Out, class F, class P> Out transform_if(my_system& s, In, In, St, Out r, F, P) { V(r); }
template <class In, class Out, class F, class Op> Out transform_inclusive_scan(my_system& s, In, In, Out r, F, Op) { V(r); }
template <class In, class Out, class F, class Op> Out transform_inclusive_scan(my_tag, In, In, Out r, F, Op) { *r = 13; return r; }
template <class In, class Out, class F, class T, class Op> Out transform_exclusive_scan(my_system& s, In, In, Out r, F, T, Op) { V(r); }
template <class It, class T> It remove(my_system& s, It f, It, const T&) { V(f); }
template <class It, class T> It remove(my_tag, It f, It, const T&) { *f = 13; return f; }
template <class In, class Out, class T> Out remove_copy(my_system& s, In, In, Out r, const T&) { V(r); }
template <class It, class St, class P> It remove_if(my_system& s, It f, It, St, P) { V(f); }
template <class It, class F> It for_each(my_system& s, It f, It, F) { V(f); }
template <class It, class F> It for_each(my_tag, It f, It, F) { *f = 13; return f; }
template <class It, class N, class F> It for_each_n(my_system& s, It f, N, F) { V(f); }
template <class A, class Bi> bool equal(my_system& s, A, A, Bi) { V(false); }
template <class A, class Bi> bool equal(my_tag, A f, A, Bi) { *f = 13; return false; }
template <class It, class T> It find(my_system& s, It f, It, const T&) { V(f); }
template <class In, class N, class Out> Out copy_n(my_system& s, In, N, Out r) { V(r); }
template <class It, class P> It remove_if(my_tag, It f, It, P) { *f = 13; return f; }
template <class In, class Out, class F> Out transform(my_tag, In, In, Out r, F) { *r = 13; return r; }
template <class It, class T> void fill(my_tag, It f, It, const T&) { *f = 13; }
template <class It, class T> void sequence(my_tag, It f, It, T, T) { *f = 13; }
template <class It, class E_> It unique(my_tag, It f, It, E_) { *f = 13; return f; }
#undef V
EXPLICIT(partition_point, BEGIN_, BEGIN_, I());
IMPLICIT(partition_point, TAGGED_, TAGGED_, I());
EXPLICIT(is_partitioned, BEGIN_, BEGIN_, I());
IMPLICIT(is_partitioned, TAGGED_, TAGGED_, I());
EXPLICIT(all_of, BEGIN_, BEGIN_, I());
IMPLICIT(all_of, TAGGED_, TAGGED_, I());
EXPLICIT(any_of, BEGIN_, BEGIN_, I());
EXPLICIT(none_of, BEGIN_, BEGIN_, I());
EXPLICIT(generate_n, BEGIN_, 1, thrust::default_random_engine());
IMPLICIT(generate_n, TAGGED_, 1, thrust::default_random_engine());
IMPLICIT(generate, TAGGED_, TAGGED_, thrust::default_random_engine());
EXPLICIT(replace_if, BEGIN_, BEGIN_, I(), 0);
IMPLICIT(replace_if, TAGGED_, TAGGED_, I(), 0);
EXPLICIT(replace, BEGIN_, BEGIN_, 0, 1);
EXPLICIT(transform_if, BEGIN_, BEGIN_, BEGIN_, thrust::negate<int>(), I());
IMPLICIT(transform_if, TAGGED_, TAGGED_, TAGGED_, thrust::negate<int>(), I());
void TestTransformIfStencilDispatchExplicit() {
  thrust::device_vector<int> vec(1);
  my_system sys(0);
  thrust::transform_if(sys, BEGIN_, BEGIN_, BEGIN_, BEGIN_, thrust::negate<int>(), I());
  ASSERT_EQUAL(true, sys.is_valid());
}
DECLARE_UNITTEST(TestTransformIfStencilDispatchExplicit);
EXPLICIT(transform_inclusive_scan, BEGIN_, BEGIN_, BEGIN_, thrust::negate<int>(), thrust::plus<int>());
IMPLICIT(transform_inclusive_scan, TAGGED_, TAGGED_, TAGGED_, thrust::negate<int>(), thrust::plus<int>());
EXPLICIT(transform_exclusive_scan, BEGIN_, BEGIN_, BEGIN_, thrust::negate<int>(), 0, thrust::plus<int>());
EXPLICIT(remove, BEGIN_, BEGIN_, 0);
IMPLICIT(remove, TAGGED_, TAGGED_, 0);
EXPLICIT(remove_copy, BEGIN_, BEGIN_, BEGIN_, 0);
void TestRemoveIfStencilDispatchExplicit() {
  thrust::device_vector<int> vec(1);
  my_system sys(0);
  thrust::remove_if(sys, BEGIN_, BEGIN_, BEGIN_, I());
  ASSERT_EQUAL(true, sys.is_valid());
}
DECLARE_UNITTEST(TestRemoveIfStencilDispatchExplicit);
EXPLICIT(for_each, BEGIN_, BEGIN_, I());
IMPLICIT(for_each, TAGGED_, TAGGED_, I());
EXPLICIT(for_each_n, BEGIN_, 1, I());
EXPLICIT(equal, BEGIN_, BEGIN_, BEGIN_);
IMPLICIT(equal, TAGGED_, TAGGED_, TAGGED_);
EXPLICIT(find, BEGIN_, BEGIN_, 0);
EXPLICIT(copy_n, BEGIN_, 1, BEGIN_);
IMPLICIT(remove_if, TAGGED_, TAGGED_, I());
IMPLICIT(transform, TAGGED_, TAGGED_, TAGGED_, thrust::negate<int>());
IMPLICIT(fill, TAGGED_, TAGGED_, 0);
IMPLICIT(sequence, TAGGED_, TAGGED_, 0, 1);
IMPLICIT(unique, TAGGED_, TAGGED_, E());

// a counting range next to a host range runs on the host (it belongs to any system); next to a
// device range, and alone, on the device
struct times_two { __host__ __device__ int operator()(int x) const { return 2 * x; } };
void TestAnySystemIteratorsFollowTheOtherRange() {
  thrust::host_vector<int> h(5);
  thrust::transform(thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(5), h.begin(), times_two());
  for (int i = 0; i < 5; i++) ASSERT_EQUAL(h[i], 2 * i);
  thrust::device_vector<int> d(5);
  thrust::transform(thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(5), d.begin(), times_two());
  ASSERT_EQUAL(d, h);
  ASSERT_EQUAL(thrust::reduce(thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(5)), 10);
  thrust::host_vector<int> c(3);
  thrust::copy(thrust::constant_iterator<int>(7), thrust::constant_iterator<int>(7) + 3, c.begin());
  ASSERT_EQUAL(c[2], 7);
  // sequence computes in the type of init and converts where it stores
  thrust::device_vector<int> q(4);
  thrust::sequence(q.begin(), q.end(), 0.5f, 1.5f);
  thrust::host_vector<int> hq = q;
  ASSERT_EQUAL(hq[0], 0); ASSERT_EQUAL(hq[1], 2); ASSERT_EQUAL(hq[2], 3); ASSERT_EQUAL(hq[3], 5);
  thrust::host_vector<int> hs(4);
  thrust::sequence(hs.begin(), hs.end(), 0.5f, 1.5f);
  ASSERT_EQUAL(hs, hq);
}
DECLARE_UNITTEST(TestAnySystemIteratorsFollowTheOtherRange);

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
