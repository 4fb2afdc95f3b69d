// The cdna4 device system's transform_reduce (the counterpart of thrust/system/cuda/detail/transform_reduce.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/transform_reduce.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/transform_reduce.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class F, class T, class Op>
T transform_reduce(const system::cdna4::execution_policy<D>& exec, It first, It last, F f, T init, Op op) {
  return system::cdna4::detail::transform_reduce_n(exec.derived(), thrust::detail::unwrap(first),
                                                   (std::int64_t)(last - first), f, init, op);
}
}}  // namespace system::cdna4
}  // namespace thrust
