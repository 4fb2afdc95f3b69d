// thrust::adjacent_difference (thrust/adjacent_difference.h;
// thrust/system/cuda/detail/adjacent_difference.h): out[0] = in[0], out[i] = op(in[i], in[i-1]).
// The output may be the input range itself: the input is then read from a temporary copy.
#pragma once
#include <numeric>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust {
namespace detail {
template <class A, class B> inline bool same_address(A, B) { return false; }
template <class T, class U> inline bool same_address(T* a, U* b) { return (const void*)a == (const void*)b; }
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/adjacent_difference.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/adjacent_difference.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class Op>
Out adjacent_difference(const detail::execution_policy_base<D>& exec, In first, In last, Out out, Op op) {
  return adjacent_difference(detail::derived_cast(detail::strip_const(exec)), first, last, out, op);
}
template <class In, class Out, class Op>
Out adjacent_difference(const system::cpp::detail::par_t&, In first, In last, Out out, Op op) {
  return std::adjacent_difference(first, last, out, op);
}
namespace detail {
template <class Policy, class In, class Out>
Out composed_adjacent_difference(const Policy& exec, In first, In last, Out out) {
  return adjacent_difference(exec, first, last, out, minus<typename detail::value_of<In>::type>());
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out>
Out adjacent_difference(execution_policy<D_>& exec, In first, In last, Out out) { return thrust::detail::composed_adjacent_difference(exec, first, last, out); }
}}  // namespace system::cdna4
template <class D_, class In, class Out>
Out adjacent_difference(const detail::execution_policy_base<D_>& exec, In first, In last, Out out) { return adjacent_difference(detail::derived_cast(detail::strip_const(exec)), first, last, out); }
template <class In, class Out>
Out adjacent_difference(const system::cpp::detail::par_t& exec, In first, In last, Out out) { return detail::composed_adjacent_difference(exec, first, last, out); }
template <class In, class Out, detail::enable_if_device<In, Out> = 0> Out adjacent_difference(In f, In l, Out o) { return adjacent_difference(typename detail::implicit_policy<In, Out>::type(), f, l, o); }
template <class In, class Out, detail::enable_if_host<In, Out> = 0> Out adjacent_difference(In f, In l, Out o) { return adjacent_difference(host, f, l, o); }
template <class In, class Out, class Op, detail::enable_if_device<In, Out, Op> = 0,
          class = typename std::iterator_traits<Out>::iterator_category>
Out adjacent_difference(In f, In l, Out o, Op op) { return adjacent_difference(typename detail::implicit_policy<In, Out, Op>::type(), f, l, o, op); }
template <class In, class Out, class Op, detail::enable_if_host<In, Out, Op> = 0,
          class = typename std::iterator_traits<Out>::iterator_category>
Out adjacent_difference(In f, In l, Out o, Op op) { return adjacent_difference(host, f, l, o, op); }
}  // namespace thrust
