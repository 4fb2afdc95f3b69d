// thrust::count / count_if (thrust/count.h): a transform_reduce of 0/1 flags.
#pragma once
#include <cstddef>
#include <thrust/transform_reduce.h>

namespace thrust {
namespace detail {
template <class F> struct flag_of {
  mutable F pred;
  template <class T> THRUST_CDNA4_HD std::ptrdiff_t operator()(const T& x) const { return pred(x) ? 1 : 0; }
};
template <class V> struct equals_value {
  V v;
  template <class T> THRUST_CDNA4_HD bool operator()(const T& x) const { return x == v; }
};
}  // namespace detail
namespace detail {
template <class Policy, class It, class Pred>
std::ptrdiff_t composed_count_if(const Policy& exec, It first, It last, Pred pred) {
  return transform_reduce(exec, first, last, detail::flag_of<Pred>{pred}, std::ptrdiff_t(0), plus<std::ptrdiff_t>());
}
}  // namespace detail
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class Pred>
std::ptrdiff_t count_if(execution_policy<D>& exec, It first, It last, Pred pred) { return thrust::detail::composed_count_if(exec.derived(), first, last, pred); }
template <class D, class It, class V>
std::ptrdiff_t count(execution_policy<D>& exec, It first, It last, const V& value) {
  return thrust::detail::composed_count_if(exec.derived(), first, last, thrust::detail::equals_value<V>{value});
}
}}  // namespace system::cdna4
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/count.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class Pred>
std::ptrdiff_t count_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return count_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <class D, class It, class V, class = typename std::iterator_traits<It>::iterator_category>
std::ptrdiff_t count(const detail::execution_policy_base<D>& exec, It first, It last, const V& value) {
  return count(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <class It, class Pred>
std::ptrdiff_t count_if(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_count_if(exec, first, last, pred); }
template <class It, class V, class = typename std::iterator_traits<It>::iterator_category>
std::ptrdiff_t count(const system::cpp::detail::par_t& exec, It first, It last, const V& value) {
  return detail::composed_count_if(exec, first, last, detail::equals_value<V>{value});
}
template <class It, class Pred, detail::enable_if_device<It, Pred> = 0> std::ptrdiff_t count_if(It f, It l, Pred p) { return count_if(typename detail::implicit_policy<It, Pred>::type(), f, l, p); }
template <class It, class Pred, detail::enable_if_host<It, Pred> = 0> std::ptrdiff_t count_if(It f, It l, Pred p) { return count_if(host, f, l, p); }
template <class It, class V, detail::enable_if_device<It, V> = 0> std::ptrdiff_t count(It f, It l, const V& v) { return count(typename detail::implicit_policy<It, V>::type(), f, l, v); }
template <class It, class V, detail::enable_if_host<It, V> = 0> std::ptrdiff_t count(It f, It l, const V& v) { return count(host, f, l, v); }
}  // namespace thrust
