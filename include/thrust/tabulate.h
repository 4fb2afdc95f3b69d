// thrust::tabulate (thrust/tabulate.h): first[i] = f(i).
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class Out, class F> struct tabulate_body {
  Out out; F f;
  THRUST_CDNA4_HD void operator()(std::int64_t i) { out[i] = f((typename std::iterator_traits<Out>::difference_type)i); }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/tabulate.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/tabulate.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class F>
void tabulate(const detail::execution_policy_base<D>& exec, It first, It last, F f) {
  tabulate(detail::derived_cast(detail::strip_const(exec)), first, last, f);
}
template <class It, class F>
void tabulate(const system::cpp::detail::par_t&, It first, It last, F f) {
  typename std::iterator_traits<It>::difference_type i = 0;
  for (; first != last; ++first, ++i) *first = f(i);
}
template <class It, class F, detail::enable_if_device<It, F> = 0> void tabulate(It f, It l, F fn) { tabulate(typename detail::implicit_policy<It, F>::type(), f, l, fn); }
template <class It, class F, detail::enable_if_host<It, F> = 0> void tabulate(It f, It l, F fn) { tabulate(host, f, l, fn); }
}  // namespace thrust
