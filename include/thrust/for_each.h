// thrust::for_each / for_each_n (thrust/for_each.h; thrust/system/cuda/detail/for_each.h).
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/system/cdna4/detail/for_each.h>
namespace thrust {

// The entry points dispatch on the policy's own type by an unqualified call, as the reference's
// do (thrust/detail/for_each.inl:32-44): the device system's overload above is found through the
// policy's base class, and a user's overload for a policy type derived from
// thrust::device_execution_policy (examples/minimal_custom_backend.cu) is preferred to it.
template <class D, class It, class F>
It for_each(const detail::execution_policy_base<D>& exec, It first, It last, F f) {
  return for_each(detail::derived_cast(detail::strip_const(exec)), first, last, f);
}
template <class D, class It, class Size, class F>
It for_each_n(const detail::execution_policy_base<D>& exec, It first, Size n, F f) {
  return for_each_n(detail::derived_cast(detail::strip_const(exec)), first, n, f);
}
template <class It, class F>
It for_each(const system::cpp::detail::par_t&, It first, It last, F f) { std::for_each(first, last, f); return last; }
template <class It, class Size, class F>
It for_each_n(const system::cpp::detail::par_t&, It first, Size n, F f) { std::for_each(first, first + n, f); return first + n; }

template <class It, class F, detail::enable_if_device<It, F> = 0> It for_each(It f, It l, F fn) { return for_each(typename detail::implicit_policy<It, F>::type(), f, l, fn); }
template <class It, class F, detail::enable_if_host<It, F> = 0> It for_each(It f, It l, F fn) { return for_each(host, f, l, fn); }
template <class It, class Size, class F, detail::enable_if_device<It, Size, F> = 0> It for_each_n(It f, Size n, F fn) { return for_each_n(typename detail::implicit_policy<It, Size, F>::type(), f, n, fn); }
template <class It, class Size, class F, detail::enable_if_host<It, Size, F> = 0> It for_each_n(It f, Size n, F fn) { return for_each_n(host, f, n, fn); }
}  // namespace thrust
