// thrust::transform_reduce (thrust/transform_reduce.h; thrust/system/cuda/detail/transform_reduce.h).
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/reduce.h>
namespace thrust {
template <class D, class It, class F, class T, class Op>
T transform_reduce(const system::cdna4::execution_policy<D>& exec, It first, It last, F f, T init, Op op) {
  return system::cdna4::detail::transform_reduce_n(exec.derived(), detail::unwrap(first),
                                                   (std::int64_t)(last - first), f, init, op);
}
template <class It, class F, class T, class Op>
T transform_reduce(const system::cpp::detail::par_t&, It first, It last, F f, T init, Op op) {
  for (; first != last; ++first) init = op(init, (T)f(*first));
  return init;
}
template <class It, class F, class T, class Op, detail::enable_if_device<It> = 0>
T transform_reduce(It f, It l, F fn, T init, Op op) { return transform_reduce(device, f, l, fn, init, op); }
template <class It, class F, class T, class Op, detail::enable_if_host<It> = 0>
T transform_reduce(It f, It l, F fn, T init, Op op) { return transform_reduce(host, f, l, fn, init, op); }
}  // namespace thrust
