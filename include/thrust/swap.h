// thrust::swap and thrust::swap_ranges (thrust/swap.h).
#pragma once
#include <algorithm>
#include <utility>
#include <thrust/detail/iterator_util.h>
#include <thrust/detail/raw_reference_cast.h>
#include <thrust/detail/swap.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
// thrust::swap(a, b) (thrust/swap.h:43-50): assignment through a temporary
template <class A, class B> THRUST_CDNA4_HD inline void swap(A& a, B& b) {
  A t = a;
  a = b;
  b = t;
}
namespace detail {
template <class A, class B> struct swap_body {
  A a; B b;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    // the elements' own swap where their type has one (testing/swap_ranges.cu:150-215)
    adl_swap(thrust::raw_reference_cast(a[i]), thrust::raw_reference_cast(b[i]));
  }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/swap_ranges.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/swap.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It1, class It2>
It2 swap_ranges(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2) {
  return swap_ranges(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2);
}
template <class It1, class It2> It2 swap_ranges(const system::cpp::detail::par_t&, It1 f1, It1 l1, It2 f2) { return std::swap_ranges(f1, l1, f2); }
template <class It1, class It2, detail::enable_if_device<It1, It2> = 0> It2 swap_ranges(It1 f1, It1 l1, It2 f2) { return swap_ranges(typename detail::implicit_policy<It1, It2>::type(), f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1, It2> = 0> It2 swap_ranges(It1 f1, It1 l1, It2 f2) { return swap_ranges(host, f1, l1, f2); }
}  // namespace thrust
