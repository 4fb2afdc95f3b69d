// thrust::transform, unary and binary (thrust/transform.h; thrust/system/cuda/detail/transform.h).
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust {
}  // namespace thrust
#include <thrust/system/cdna4/detail/transform.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/transform.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class F>
Out transform(const detail::execution_policy_base<D>& exec, In first, In last, Out out, F f) {
  return transform(detail::derived_cast(detail::strip_const(exec)), first, last, out, f);
}
template <class D, class In1, class In2, class Out, class F>
Out transform(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, Out out, F f) {
  return transform(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, out, f);
}
template <class In, class Out, class F>
Out transform(const system::cpp::detail::par_t&, In first, In last, Out out, F f) { return std::transform(first, last, out, f); }
template <class In1, class In2, class Out, class F>
Out transform(const system::cpp::detail::par_t&, In1 first1, In1 last1, In2 first2, Out out, F f) {
  return std::transform(first1, last1, first2, out, f);
}

template <class In, class Out, class F, detail::enable_if_device<In> = 0>
Out transform(In f, In l, Out o, F fn) { return transform(device, f, l, o, fn); }
template <class In, class Out, class F, detail::enable_if_host<In> = 0>
Out transform(In f, In l, Out o, F fn) { return transform(host, f, l, o, fn); }
template <class In1, class In2, class Out, class F, detail::enable_if_device<In1> = 0,
          class = typename std::iterator_traits<In2>::iterator_category>
Out transform(In1 f, In1 l, In2 f2, Out o, F fn) { return transform(device, f, l, f2, o, fn); }
template <class In1, class In2, class Out, class F, detail::enable_if_host<In1> = 0,
          class = typename std::iterator_traits<In2>::iterator_category>
Out transform(In1 f, In1 l, In2 f2, Out o, F fn) { return transform(host, f, l, f2, o, fn); }
}  // namespace thrust
