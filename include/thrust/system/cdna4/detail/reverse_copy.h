// The cdna4 device system's reverse_copy (the counterpart of thrust/system/cuda/detail/reverse_copy.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/reverse.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/reverse.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out>
Out reverse_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out result) {
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::for_each_index(
      exec.derived(), n,
      thrust::detail::reverse_copy_body<typename thrust::detail::unwrap_iterator<In>::type, typename thrust::detail::unwrap_iterator<Out>::type>{thrust::detail::unwrap(first), thrust::detail::unwrap(result), n},
      "reverse_copy: failed to synchronize");
  return result + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
