// The cdna4 device system's reverse (the counterpart of thrust/system/cuda/detail/reverse.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/reverse.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/reverse.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It>
void reverse(const system::cdna4::execution_policy<D>& exec, It first, It last) {
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::for_each_index(exec.derived(), n / 2, thrust::detail::reverse_body<typename thrust::detail::unwrap_iterator<It>::type>{thrust::detail::unwrap(first), n},
                                        "reverse: failed to synchronize");
}
}}  // namespace system::cdna4
}  // namespace thrust
