// thrust::uninitialized_copy / uninitialized_copy_n (thrust/uninitialized_copy.h).  Device ranges
// hold trivially copyable elements, for which construction is assignment.
#pragma once
#include <memory>
#include <thrust/copy.h>
#include <thrust/system/cdna4/detail/uninitialized_copy.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/uninitialized_copy.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out>
Out uninitialized_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  return uninitialized_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <class In, class Out>
Out uninitialized_copy(const system::cpp::detail::par_t&, In first, In last, Out result) { return std::uninitialized_copy(first, last, result); }
namespace detail {
template <class Policy, class In, class Size, class Out>
Out composed_uninitialized_copy_n(const Policy& exec, In first, Size n, Out result) { return uninitialized_copy(exec, first, first + n, result); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Size, class Out>
Out uninitialized_copy_n(execution_policy<D_>& exec, In first, Size n, Out result) { return thrust::detail::composed_uninitialized_copy_n(exec, first, n, result); }
}}  // namespace system::cdna4
template <class D_, class In, class Size, class Out>
Out uninitialized_copy_n(const detail::execution_policy_base<D_>& exec, In first, Size n, Out result) { return uninitialized_copy_n(detail::derived_cast(detail::strip_const(exec)), first, n, result); }
template <class In, class Size, class Out>
Out uninitialized_copy_n(const system::cpp::detail::par_t& exec, In first, Size n, Out result) { return detail::composed_uninitialized_copy_n(exec, first, n, result); }
// without a policy: iterators retagged with a user's policy type select that policy
// (testing/uninitialized_copy.cu:37-100); any other pair of ranges is a copy between their systems
template <class In, class Out, typename std::enable_if<!detail::has_user_policy<In, Out>::value, int>::type = 0>
Out uninitialized_copy(In f, In l, Out o) { return copy(f, l, o); }
template <class In, class Out, typename std::enable_if<detail::has_user_policy<In, Out>::value, int>::type = 0>
Out uninitialized_copy(In f, In l, Out o) { return uninitialized_copy(typename detail::implicit_policy<In, Out>::type(), f, l, o); }
template <class In, class Size, class Out, class = typename std::iterator_traits<In>::iterator_category,
          typename std::enable_if<!detail::has_user_policy<In, Out>::value, int>::type = 0>
Out uninitialized_copy_n(In f, Size n, Out o) { return copy(f, f + n, o); }
template <class In, class Size, class Out, class = typename std::iterator_traits<In>::iterator_category,
          typename std::enable_if<detail::has_user_policy<In, Out>::value, int>::type = 0>
Out uninitialized_copy_n(In f, Size n, Out o) { return uninitialized_copy_n(typename detail::implicit_policy<In, Out>::type(), f, n, o); }
}  // namespace thrust
