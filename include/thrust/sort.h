// thrust::sort / stable_sort / sort_by_key / stable_sort_by_key (thrust/sort.h:77-925).
// Device ranges (device_vector iterators, device_ptr, or raw pointers under a device policy)
// go to the radix-sort kernels; host ranges are sorted on the host.
#pragma once
#include <cstring>
#include <thrust/system/cdna4/detail/index_algorithms.h>
#include <algorithm>
#include <numeric>
#include <vector>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/algorithms.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>
#include <thrust/system/detail/sequential/algorithms.h>

namespace thrust {

// ---- device, explicit policy ---------------------------------------------------------
namespace detail {
// a contiguous device range (device_ptr or raw pointer), as opposed to a fancy iterator
template <class It> struct is_contiguous_device : std::is_pointer<typename unwrap_iterator<It>::type> {};

template <class Policy, class It, class Compare>
void sort_range(const Policy& exec, It first, It last, Compare comp, std::true_type) {
  system::cdna4::detail::sort_keys(exec, unwrap(first), (std::int64_t)(last - first), comp);
}
// A fancy range (zip, permutation, ...) is sorted in a contiguous temporary of its value type and
// written back.
template <class Policy, class It, class Compare>
void sort_range(const Policy& exec, It first, It last, Compare comp, std::false_type) {
  namespace sd = system::cdna4::detail;
  typedef typename value_of<It>::type T;
  const std::int64_t n = (std::int64_t)(last - first);
  if (n <= 0) return;
  const sd::execute_on_stream inner(sd::stream_of(exec), false);  // same stream, no waits in between
  sd::temporary_storage tmp((std::size_t)n * sizeof(T), exec);
  T* p = static_cast<T*>(tmp.data());
  sd::transform_n(inner, unwrap(first), p, n, identity<T>());
  sd::sort_keys(inner, p, n, comp);
  sd::transform_n(exec, p, unwrap(first), n, identity<T>());
}

template <class K, class U> K* pick_keys(U* contiguous, void*) { return const_cast<K*>(static_cast<const K*>(contiguous)); }
template <class K, class It> K* pick_keys(It, void* temporary) { return static_cast<K*>(temporary); }
template <class Policy, class KIt, class VIt, class Compare>
void sort_pairs_range(const Policy& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp, std::true_type) {
  system::cdna4::detail::sort_pairs(exec, unwrap(kfirst), unwrap(vfirst), (std::int64_t)(klast - kfirst), comp);
}
// Fancy keys or values (typically a zip_iterator of several value arrays): the keys are sorted
// together with their positions, then the values are permuted through a temporary.
template <class Policy, class KIt, class VIt, class Compare>
void sort_pairs_range(const Policy& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp, std::false_type) {
  namespace sd = system::cdna4::detail;
  typedef typename value_of<KIt>::type K;
  typedef typename value_of<VIt>::type V;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  if (n <= 0) return;
  if (n >= (std::int64_t(1) << 32) - 1) sd::throw_on_error(1, "sort_by_key: more than 2^32 - 2 elements");
  const sd::execute_on_stream inner(sd::stream_of(exec), false);
  sd::temporary_storage index_bytes((std::size_t)n * sizeof(std::uint32_t), exec);
  std::uint32_t* index = static_cast<std::uint32_t*>(index_bytes.data());
  sd::sequence_n(inner, index, n, std::uint32_t(0), std::uint32_t(1));
  {
    sd::temporary_storage key_bytes(is_contiguous_device<KIt>::value ? 0 : (std::size_t)n * sizeof(K), exec);
    K* keys = pick_keys<K>(unwrap(kfirst), key_bytes.data());
    if (!is_contiguous_device<KIt>::value) sd::transform_n(inner, unwrap(kfirst), keys, n, identity<K>());
    sd::sort_pairs(inner, keys, index, n, comp);
    if (!is_contiguous_device<KIt>::value) sd::transform_n(inner, keys, unwrap(kfirst), n, identity<K>());
  }
  sd::temporary_storage value_bytes((std::size_t)n * sizeof(V), exec);
  V* moved = static_cast<V*>(value_bytes.data());
  sd::gather_n(inner, unwrap(vfirst), index, moved, n);
  sd::transform_n(exec, moved, unwrap(vfirst), n, identity<V>());
}
}  // namespace detail

template <class D, class It, class Compare> void stable_sort(const detail::execution_policy_base<D>& exec, It first, It last, Compare comp);
template <class D, class It> void stable_sort(const detail::execution_policy_base<D>& exec, It first, It last);
template <class D, class KIt, class VIt, class Compare>
void stable_sort_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp);
template <class D, class KIt, class VIt> void stable_sort_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst);
}  // namespace thrust
#include <thrust/system/cdna4/detail/sort.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/sort.inl:32-44, :84-100):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class Compare>
void stable_sort(const detail::execution_policy_base<D>& exec, It first, It last, Compare comp) {
  stable_sort(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <class D, class It>
void stable_sort(const detail::execution_policy_base<D>& exec, It first, It last) {
  stable_sort(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <class D, class It, class Compare>
void sort(const detail::execution_policy_base<D>& exec, It first, It last, Compare comp) {
  sort(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <class D, class It>
void sort(const detail::execution_policy_base<D>& exec, It first, It last) {
  sort(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <class D, class KIt, class VIt, class Compare>
void stable_sort_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  stable_sort_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, comp);
}
template <class D, class KIt, class VIt>
void stable_sort_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst) {
  stable_sort_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst);
}
template <class D, class KIt, class VIt, class Compare>
void sort_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  sort_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, comp);
}
template <class D, class KIt, class VIt>
void sort_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst) {
  sort_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst);
}

// ---- host, explicit policy -----------------------------------------------------------
namespace detail {
// Floating-point keys under less / greater sort by their radix encoding, as the reference's host
// system does (thrust/system/detail/sequential/stable_radix_sort.inl:43-139: negatives with all
// bits flipped, the others with the sign bit flipped): a total order in which -0 comes before +0
// and NaNs take the place of their bit patterns — `a < b` on floats is not an ordering when NaNs
// are present and would leave -0 / +0 in input order.
inline std::uint32_t radix_key(float f) {
  std::uint32_t u;
  std::memcpy(&u, &f, sizeof u);
  return u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
inline std::uint64_t radix_key(double f) {
  std::uint64_t u;
  std::memcpy(&u, &f, sizeof u);
  return u ^ ((u >> 63) ? 0xFFFFFFFFFFFFFFFFull : 0x8000000000000000ull);
}
template <class K, class Compare, bool Encoded = std::is_floating_point<K>::value && (system::cdna4::detail::order_code<Compare>::value >= 0)>
struct host_order {
  mutable Compare comp;
  bool operator()(const K& a, const K& b) const { return comp(a, b); }
};
template <class K, class Compare>
struct host_order<K, Compare, true> {
  Compare comp;
  bool operator()(const K& a, const K& b) const {
    return system::cdna4::detail::order_code<Compare>::value == 0 ? radix_key(a) < radix_key(b) : radix_key(a) > radix_key(b);
  }
};
}  // namespace detail
template <class It, class Compare>
void stable_sort(const system::cpp::detail::par_t&, It first, It last, Compare comp) {
  typedef typename detail::value_of<It>::type K;
  std::stable_sort(first, last, detail::host_order<K, Compare>{comp});
}
template <class It>
void stable_sort(const system::cpp::detail::par_t& e, It first, It last) { stable_sort(e, first, last, less<typename detail::value_of<It>::type>()); }
template <class It, class Compare>
void sort(const system::cpp::detail::par_t& e, It first, It last, Compare comp) { stable_sort(e, first, last, comp); }
template <class It>
void sort(const system::cpp::detail::par_t& e, It first, It last) { stable_sort(e, first, last); }
template <class KIt, class VIt, class Compare>
void stable_sort_by_key(const system::cpp::detail::par_t&, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  typedef typename detail::value_of<KIt>::type K;
  typedef typename detail::value_of<VIt>::type V;
  const std::size_t n = (std::size_t)(klast - kfirst);
  std::vector<std::size_t> idx(n);
  std::iota(idx.begin(), idx.end(), std::size_t(0));
  std::vector<K> k(kfirst, klast);
  std::vector<V> v(vfirst, vfirst + n);
  const detail::host_order<K, Compare> order{comp};
  std::stable_sort(idx.begin(), idx.end(), [&](std::size_t a, std::size_t b) { return order(k[a], k[b]); });
  for (std::size_t i = 0; i < n; i++) { kfirst[i] = k[idx[i]]; vfirst[i] = v[idx[i]]; }
}
template <class KIt, class VIt>
void stable_sort_by_key(const system::cpp::detail::par_t& e, KIt kfirst, KIt klast, VIt vfirst) {
  stable_sort_by_key(e, kfirst, klast, vfirst, less<typename detail::value_of<KIt>::type>());
}
template <class KIt, class VIt, class Compare>
void sort_by_key(const system::cpp::detail::par_t& e, KIt kfirst, KIt klast, VIt vfirst, Compare comp) { stable_sort_by_key(e, kfirst, klast, vfirst, comp); }
template <class KIt, class VIt>
void sort_by_key(const system::cpp::detail::par_t& e, KIt kfirst, KIt klast, VIt vfirst) { stable_sort_by_key(e, kfirst, klast, vfirst); }

// ---- no policy: the iterator's system decides (thrust/detail/sort.inl:202-339) --------
#define THRUST_CDNA4_SORT_DISPATCH(NAME)                                                                         \
  template <class It, detail::enable_if_device<It> = 0> void NAME(It f, It l) { NAME(typename detail::implicit_policy<It>::type(), f, l); }              \
  template <class It, class C, detail::enable_if_device<It, C> = 0> void NAME(It f, It l, C c) { NAME(typename detail::implicit_policy<It>::type(), f, l, c); } \
  template <class It, detail::enable_if_host<It> = 0> void NAME(It f, It l) { NAME(host, f, l); }                  \
  template <class It, class C, detail::enable_if_host<It, C> = 0> void NAME(It f, It l, C c) { NAME(host, f, l, c); }
THRUST_CDNA4_SORT_DISPATCH(sort)
THRUST_CDNA4_SORT_DISPATCH(stable_sort)
#undef THRUST_CDNA4_SORT_DISPATCH
#define THRUST_CDNA4_SORT_BY_KEY_DISPATCH(NAME)                                                                  \
  template <class K, class V, detail::enable_if_device<K, V> = 0> void NAME(K f, K l, V v) { NAME(typename detail::implicit_policy<K>::type(), f, l, v); }  \
  template <class K, class V, class C, detail::enable_if_device<K, V, C> = 0> void NAME(K f, K l, V v, C c) { NAME(typename detail::implicit_policy<K>::type(), f, l, v, c); } \
  template <class K, class V, detail::enable_if_host<K, V> = 0> void NAME(K f, K l, V v) { NAME(host, f, l, v); }      \
  template <class K, class V, class C, detail::enable_if_host<K, V, C> = 0> void NAME(K f, K l, V v, C c) { NAME(host, f, l, v, c); }
THRUST_CDNA4_SORT_BY_KEY_DISPATCH(sort_by_key)
THRUST_CDNA4_SORT_BY_KEY_DISPATCH(stable_sort_by_key)
#undef THRUST_CDNA4_SORT_BY_KEY_DISPATCH


// ---------------------------------------------------------------------------------------
// is_sorted / is_sorted_until (thrust/sort.h:1160-): the first position whose element is before
// its predecessor, as a minimum over such positions.
// ---------------------------------------------------------------------------------------
namespace detail {
template <class It, class Compare> struct descent_index {
  It p; mutable Compare comp; std::int64_t n;
  THRUST_CDNA4_HD std::int64_t operator()(std::int64_t i) const { return comp(p[i + 1], p[i]) ? i + 1 : n; }
};
struct min_position {
  THRUST_CDNA4_HD std::int64_t operator()(std::int64_t a, std::int64_t b) const { return a < b ? a : b; }
};
}  // namespace detail
template <class D, class It, class Compare>
It is_sorted_until(const system::cdna4::execution_policy<D>& exec, It first, It last, Compare comp) {
  const std::int64_t n = (std::int64_t)(last - first);
  if (n < 2) return last;
  const std::int64_t at = system::cdna4::detail::reduce_index(
      exec.derived(), n - 1, detail::descent_index<typename detail::unwrap_iterator<It>::type, Compare>{detail::unwrap(first), comp, n}, n,
      detail::min_position());
  return first + at;
}
template <class It, class Compare>
It is_sorted_until(const system::cpp::detail::par_t&, It first, It last, Compare comp) { return std::is_sorted_until(first, last, comp); }
namespace detail {
template <class Policy, class It>
It composed_is_sorted_until(const Policy& exec, It first, It last) { return is_sorted_until(exec, first, last, less<>()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It>
It is_sorted_until(execution_policy<D_>& exec, It first, It last) { return thrust::detail::composed_is_sorted_until(exec, first, last); }
}}  // namespace system::cdna4
template <class D_, class It>
It is_sorted_until(const detail::execution_policy_base<D_>& exec, It first, It last) { return is_sorted_until(detail::derived_cast(detail::strip_const(exec)), first, last); }
template <class It>
It is_sorted_until(const system::cpp::detail::par_t& exec, It first, It last) { return detail::composed_is_sorted_until(exec, first, last); }
namespace detail {
template <class Policy, class It, class Compare>
bool composed_is_sorted(const Policy& exec, It first, It last, Compare comp) { return is_sorted_until(exec, first, last, comp) == last; }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Compare>
bool is_sorted(execution_policy<D_>& exec, It first, It last, Compare comp) { return thrust::detail::composed_is_sorted(exec, first, last, comp); }
}}  // namespace system::cdna4
template <class D_, class It, class Compare>
bool is_sorted(const detail::execution_policy_base<D_>& exec, It first, It last, Compare comp) { return is_sorted(detail::derived_cast(detail::strip_const(exec)), first, last, comp); }
template <class It, class Compare>
bool is_sorted(const system::cpp::detail::par_t& exec, It first, It last, Compare comp) { return detail::composed_is_sorted(exec, first, last, comp); }
namespace detail {
template <class Policy, class It>
bool composed_is_sorted(const Policy& exec, It first, It last) { return is_sorted_until(exec, first, last, less<>()) == last; }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It>
bool is_sorted(execution_policy<D_>& exec, It first, It last) { return thrust::detail::composed_is_sorted(exec, first, last); }
}}  // namespace system::cdna4
template <class D_, class It>
bool is_sorted(const detail::execution_policy_base<D_>& exec, It first, It last) { return is_sorted(detail::derived_cast(detail::strip_const(exec)), first, last); }
template <class It>
bool is_sorted(const system::cpp::detail::par_t& exec, It first, It last) { return detail::composed_is_sorted(exec, first, last); }
template <class It, detail::enable_if_device<It> = 0> It is_sorted_until(It f, It l) { return is_sorted_until(typename detail::implicit_policy<It>::type(), f, l); }
template <class It, detail::enable_if_host<It> = 0> It is_sorted_until(It f, It l) { return is_sorted_until(host, f, l); }
template <class It, class C, detail::enable_if_device<It, C> = 0> It is_sorted_until(It f, It l, C c) { return is_sorted_until(typename detail::implicit_policy<It, C>::type(), f, l, c); }
template <class It, class C, detail::enable_if_host<It, C> = 0> It is_sorted_until(It f, It l, C c) { return is_sorted_until(host, f, l, c); }
template <class It, detail::enable_if_device<It> = 0> bool is_sorted(It f, It l) { return is_sorted(typename detail::implicit_policy<It>::type(), f, l); }
template <class It, detail::enable_if_host<It> = 0> bool is_sorted(It f, It l) { return is_sorted(host, f, l); }
template <class It, class C, detail::enable_if_device<It, C> = 0> bool is_sorted(It f, It l, C c) { return is_sorted(typename detail::implicit_policy<It, C>::type(), f, l, c); }
template <class It, class C, detail::enable_if_host<It, C> = 0> bool is_sorted(It f, It l, C c) { return is_sorted(host, f, l, c); }
}  // namespace thrust
