// The cdna4 device system's replace (the counterpart of thrust/system/cuda/detail/replace.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/replace.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/replace.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class S, class Out, class Pred, class T>
Out replace_copy_if(const system::cdna4::execution_policy<D>& exec, In first, In last, S stencil, Out result, Pred pred, const T& value) {
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::for_each_index(
      exec.derived(), n,
      thrust::detail::replace_body<typename thrust::detail::unwrap_iterator<In>::type, typename thrust::detail::unwrap_iterator<S>::type,
                           typename thrust::detail::unwrap_iterator<Out>::type, Pred, T>{thrust::detail::unwrap(first), thrust::detail::unwrap(stencil), thrust::detail::unwrap(result), pred, value},
      "replace: failed to synchronize");
  return result + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
