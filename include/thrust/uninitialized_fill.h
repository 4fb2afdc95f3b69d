// thrust::uninitialized_fill / uninitialized_fill_n (thrust/uninitialized_fill.h).  Device
// ranges hold trivially copyable elements, for which construction is assignment
// (thrust/system/detail/generic/uninitialized_fill.inl takes the same shortcut).
#pragma once
#include <memory>
#include <thrust/fill.h>
#include <thrust/system/cdna4/detail/uninitialized_fill.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/uninitialized_fill.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class T>
void uninitialized_fill(const detail::execution_policy_base<D>& exec, It first, It last, const T& x) {
  uninitialized_fill(detail::derived_cast(detail::strip_const(exec)), first, last, x);
}
template <class It, class T>
void uninitialized_fill(const system::cpp::detail::par_t&, It first, It last, const T& x) { std::uninitialized_fill(first, last, x); }
namespace detail {
template <class Policy, class It, class Size, class T>
It composed_uninitialized_fill_n(const Policy& exec, It first, Size n, const T& x) {
  uninitialized_fill(exec, first, first + n, x);
  return first + n;
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Size, class T>
It uninitialized_fill_n(execution_policy<D_>& exec, It first, Size n, const T& x) { return thrust::detail::composed_uninitialized_fill_n(exec, first, n, x); }
}}  // namespace system::cdna4
template <class D_, class It, class Size, class T>
It uninitialized_fill_n(const detail::execution_policy_base<D_>& exec, It first, Size n, const T& x) { return uninitialized_fill_n(detail::derived_cast(detail::strip_const(exec)), first, n, x); }
template <class It, class Size, class T>
It uninitialized_fill_n(const system::cpp::detail::par_t& exec, It first, Size n, const T& x) { return detail::composed_uninitialized_fill_n(exec, first, n, x); }
template <class It, class T, detail::enable_if_device<It, T> = 0> void uninitialized_fill(It f, It l, const T& x) { uninitialized_fill(typename detail::implicit_policy<It, T>::type(), f, l, x); }
template <class It, class T, detail::enable_if_host<It, T> = 0> void uninitialized_fill(It f, It l, const T& x) { uninitialized_fill(host, f, l, x); }
template <class It, class Size, class T, detail::enable_if_device<It, Size, T> = 0> It uninitialized_fill_n(It f, Size n, const T& x) { return uninitialized_fill_n(typename detail::implicit_policy<It, Size, T>::type(), f, n, x); }
template <class It, class Size, class T, detail::enable_if_host<It, Size, T> = 0> It uninitialized_fill_n(It f, Size n, const T& x) { return uninitialized_fill_n(host, f, n, x); }
}  // namespace thrust
