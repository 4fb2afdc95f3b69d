// thrust::transform_reduce (thrust/transform_reduce.h; thrust/system/cuda/detail/transform_reduce.h).
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/reduce.h>
#include <thrust/system/cdna4/detail/transform_reduce.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/transform_reduce.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class F, class T, class Op>
T transform_reduce(const detail::execution_policy_base<D>& exec, It first, It last, F f, T init, Op op) {
  return transform_reduce(detail::derived_cast(detail::strip_const(exec)), first, last, f, init, op);
}
template <class It, class F, class T, class Op>
T transform_reduce(const system::cpp::detail::par_t&, It first, It last, F f, T init, Op op) {
  for (; first != last; ++first) init = op(init, (T)f(*first));
  return init;
}
template <class It, class F, class T, class Op, detail::enable_if_device<It, F, T, Op> = 0>
T transform_reduce(It f, It l, F fn, T init, Op op) { return transform_reduce(typename detail::implicit_policy<It, F, T, Op>::type(), f, l, fn, init, op); }
template <class It, class F, class T, class Op, detail::enable_if_host<It, F, T, Op> = 0>
T transform_reduce(It f, It l, F fn, T init, Op op) { return transform_reduce(host, f, l, fn, init, op); }
}  // namespace thrust
