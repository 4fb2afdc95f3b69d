// thrust::fill / fill_n (thrust/fill.h; thrust/system/cuda/detail/fill.h:61-75).  Contiguous
// device ranges of 1-, 2-, 4- and 8-byte elements go to the library's typed fill kernel (no
// device compiler needed in the caller); other element sizes and fancy outputs instantiate a
// kernel template.
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust {
namespace detail {
template <class T> struct fill_value {
  T v;
  template <class U> THRUST_CDNA4_HD T operator()(const U&) const { return v; }
};
template <class Policy, class T, class V>
typename std::enable_if<sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8>::type
fill_device(const Policy& exec, device_ptr<T> first, std::int64_t n, const V& value) {
  namespace sd = system::cdna4::detail;
  const T v = static_cast<T>(value);
  if (n <= 0) return;
  sd::throw_on_error(thrust_cdna4_fill(first.get(), &v, (int)sizeof(T), n, sd::stream_of(exec)), "fill");
  sd::synchronize_optional(exec, "fill: failed to synchronize");
}
template <class Policy, class T, class V>
typename std::enable_if<!(sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8)>::type
fill_device(const Policy& exec, device_ptr<T> first, std::int64_t n, const V& value) {
  system::cdna4::detail::transform_n(exec, first.get(), first.get(), n, fill_value<T>{static_cast<T>(value)});
}
template <class Policy, class Out, class V>
void fill_device(const Policy& exec, Out first, std::int64_t n, const V& value) {  // fancy output
  typedef typename value_of<Out>::type T;
  system::cdna4::detail::transform_n(exec, unwrap(first), unwrap(first), n, fill_value<T>{static_cast<T>(value)});
}
}  // namespace detail

}  // namespace thrust
#include <thrust/system/cdna4/detail/fill.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/fill.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class V>
void fill(const detail::execution_policy_base<D>& exec, It first, It last, const V& value) {
  fill(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <class It, class V>
void fill(const system::cpp::detail::par_t&, It first, It last, const V& value) { std::fill(first, last, value); }
namespace detail {
template <class Policy, class It, class Size, class V>
It composed_fill_n(const Policy& exec, It first, Size n, const V& value) {
  fill(exec, first, first + n, value);
  return first + n;
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Size, class V>
It fill_n(execution_policy<D_>& exec, It first, Size n, const V& value) { return thrust::detail::composed_fill_n(exec, first, n, value); }
}}  // namespace system::cdna4
template <class D_, class It, class Size, class V>
It fill_n(const detail::execution_policy_base<D_>& exec, It first, Size n, const V& value) { return fill_n(detail::derived_cast(detail::strip_const(exec)), first, n, value); }
template <class It, class Size, class V>
It fill_n(const system::cpp::detail::par_t& exec, It first, Size n, const V& value) { return detail::composed_fill_n(exec, first, n, value); }
template <class It, class V, detail::enable_if_device<It, V> = 0> void fill(It f, It l, const V& v) { fill(typename detail::implicit_policy<It, V>::type(), f, l, v); }
template <class It, class V, detail::enable_if_host<It, V> = 0> void fill(It f, It l, const V& v) { fill(host, f, l, v); }
template <class It, class Size, class V, detail::enable_if_device<It, Size, V> = 0> It fill_n(It f, Size n, const V& v) { return fill_n(typename detail::implicit_policy<It, Size, V>::type(), f, n, v); }
template <class It, class Size, class V, detail::enable_if_host<It, Size, V> = 0> It fill_n(It f, Size n, const V& v) { return fill_n(host, f, n, v); }
}  // namespace thrust
