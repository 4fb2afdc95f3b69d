// thrust::reverse / reverse_copy (thrust/reverse.h).
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class It> struct reverse_body {
  It p; std::int64_t n;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    typename std::iterator_traits<It>::value_type a = p[i], b = p[n - 1 - i];
    p[i] = b;
    p[n - 1 - i] = a;
  }
};
template <class In, class Out> struct reverse_copy_body {
  In in; Out out; std::int64_t n;
  THRUST_CDNA4_HD void operator()(std::int64_t i) { out[i] = in[n - 1 - i]; }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/reverse.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/reverse.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It>
void reverse(const detail::execution_policy_base<D>& exec, It first, It last) {
  reverse(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <class It> void reverse(const system::cpp::detail::par_t&, It first, It last) { std::reverse(first, last); }
}  // namespace thrust
#include <thrust/system/cdna4/detail/reverse_copy.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/reverse.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out>
Out reverse_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  return reverse_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <class In, class Out> Out reverse_copy(const system::cpp::detail::par_t&, In first, In last, Out result) { return std::reverse_copy(first, last, result); }
template <class It, detail::enable_if_device<It> = 0> void reverse(It f, It l) { reverse(typename detail::implicit_policy<It>::type(), f, l); }
template <class It, detail::enable_if_host<It> = 0> void reverse(It f, It l) { reverse(host, f, l); }
template <class In, class Out, detail::enable_if_device<In, Out> = 0> Out reverse_copy(In f, In l, Out o) { return reverse_copy(typename detail::implicit_policy<In, Out>::type(), f, l, o); }
template <class In, class Out, detail::enable_if_host<In, Out> = 0> Out reverse_copy(In f, In l, Out o) { return reverse_copy(host, f, l, o); }
}  // namespace thrust
