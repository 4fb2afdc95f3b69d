// The cdna4 device system's swap_ranges (the counterpart of thrust/system/cuda/detail/swap_ranges.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/swap.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/swap.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It1, class It2>
It2 swap_ranges(const system::cdna4::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2) {
  const std::int64_t n = (std::int64_t)(last1 - first1);
  system::cdna4::detail::for_each_index(
      exec.derived(), n,
      thrust::detail::swap_body<typename thrust::detail::unwrap_iterator<It1>::type, typename thrust::detail::unwrap_iterator<It2>::type>{thrust::detail::unwrap(first1), thrust::detail::unwrap(first2)},
      "swap_ranges: failed to synchronize");
  return first2 + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
