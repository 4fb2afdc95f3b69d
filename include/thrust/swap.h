// thrust::swap and thrust::swap_ranges (thrust/swap.h).
#pragma once
#include <algorithm>
#include <utility>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
template <class A, class B> THRUST_CDNA4_HD inline void swap(A& a, B& b) {
  A t = a;
  a = b;
  b = t;
}
namespace detail {
template <class A, class B> struct swap_body {
  A a; B b;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    typename std::iterator_traits<A>::value_type t = a[i];
    a[i] = b[i];
    b[i] = t;
  }
};
}  // namespace detail
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It1, class It2>
It2 swap_ranges(const system::cdna4::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2) {
  const std::int64_t n = (std::int64_t)(last1 - first1);
  system::cdna4::detail::for_each_index(
      exec.derived(), n,
      thrust::detail::swap_body<typename thrust::detail::unwrap_iterator<It1>::type, typename thrust::detail::unwrap_iterator<It2>::type>{thrust::detail::unwrap(first1), thrust::detail::unwrap(first2)},
      "swap_ranges: failed to synchronize");
  return first2 + n;
}
}}  // namespace system::cdna4
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/swap.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It1, class It2>
It2 swap_ranges(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2) {
  return swap_ranges(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2);
}
template <class It1, class It2> It2 swap_ranges(const system::cpp::detail::par_t&, It1 f1, It1 l1, It2 f2) { return std::swap_ranges(f1, l1, f2); }
template <class It1, class It2, detail::enable_if_device<It1> = 0> It2 swap_ranges(It1 f1, It1 l1, It2 f2) { return swap_ranges(device, f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1> = 0> It2 swap_ranges(It1 f1, It1 l1, It2 f2) { return swap_ranges(host, f1, l1, f2); }
}  // namespace thrust
