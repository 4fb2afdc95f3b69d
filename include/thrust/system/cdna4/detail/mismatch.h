// The cdna4 device system's mismatch (the counterpart of thrust/system/cuda/detail/mismatch.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/mismatch.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/mismatch.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It1, class It2, class Pred>
pair<It1, It2> mismatch(const system::cdna4::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, Pred pred) {
  const std::int64_t n = (std::int64_t)(last1 - first1);
  const std::int64_t at = system::cdna4::detail::reduce_index(
      exec.derived(), n,
      thrust::detail::differ_index<typename thrust::detail::unwrap_iterator<It1>::type, typename thrust::detail::unwrap_iterator<It2>::type, Pred>{
          thrust::detail::unwrap(first1), thrust::detail::unwrap(first2), pred, n},
      n, thrust::detail::min_index());
  return thrust::make_pair(first1 + at, first2 + at);
}
}}  // namespace system::cdna4
}  // namespace thrust
