// The cdna4 device system's reduce (the counterpart of thrust/system/cuda/detail/reduce.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/reduce.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/reduce.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// ---------------------------------------------------------------------------------------
// reduce
// ---------------------------------------------------------------------------------------
template <class D, class It, class T, class Op>
T reduce(const system::cdna4::execution_policy<D>& exec, It first, It last, T init, Op op) {
  typedef typename thrust::detail::value_of<It>::type V;
  return system::cdna4::detail::transform_reduce_n(exec.derived(), thrust::detail::unwrap(first),
                                                   (std::int64_t)(last - first), identity<V>(), init, op);
}
template <class D, class It, class T>
T reduce(const system::cdna4::execution_policy<D>& exec, It first, It last, T init) { return reduce(exec, first, last, init, plus<T>()); }
template <class D, class It>
typename thrust::detail::value_of<It>::type reduce(const system::cdna4::execution_policy<D>& exec, It first, It last) {
  typedef typename thrust::detail::value_of<It>::type V;
  return reduce(exec, first, last, V(0), plus<V>());
}
}}  // namespace system::cdna4
}  // namespace thrust
