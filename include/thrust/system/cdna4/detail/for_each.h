// The cdna4 device system's for_each (the counterpart of thrust/system/cuda/detail/for_each.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/for_each.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/for_each.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementation, found through the policy's type
template <class D, class It, class F>
It for_each(const execution_policy<D>& exec, It first, It last, F f) {
  detail::apply_n(exec.derived(), thrust::detail::unwrap(first), (std::int64_t)(last - first), f);
  return last;
}
template <class D, class It, class Size, class F>
It for_each_n(const execution_policy<D>& exec, It first, Size n, F f) {
  detail::apply_n(exec.derived(), thrust::detail::unwrap(first), (std::int64_t)n, f);
  return first + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
