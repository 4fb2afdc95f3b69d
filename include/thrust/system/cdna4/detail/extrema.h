// The cdna4 device system's extrema (the counterpart of thrust/system/cuda/detail/extrema.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/extrema.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/extrema.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class Compare>
It min_element(const system::cdna4::execution_policy<D>& exec, It first, It last, Compare comp) {
  if (first == last) return last;
  return first + thrust::detail::extrema_of(exec.derived(), first, last, comp).lo_at;
}
template <class D, class It, class Compare>
It max_element(const system::cdna4::execution_policy<D>& exec, It first, It last, Compare comp) {
  if (first == last) return last;
  return first + thrust::detail::extrema_of(exec.derived(), first, last, comp).hi_at;
}
template <class D, class It, class Compare>
pair<It, It> minmax_element(const system::cdna4::execution_policy<D>& exec, It first, It last, Compare comp) {
  if (first == last) return thrust::make_pair(last, last);
  const auto e = thrust::detail::extrema_of(exec.derived(), first, last, comp);
  return thrust::make_pair(first + e.lo_at, first + e.hi_at);
}
// without a comparison: operator< (thrust/extrema.h:79-81, :348-350, :606-608)
template <class D, class It>
It min_element(const system::cdna4::execution_policy<D>& exec, It first, It last) { return min_element(exec, first, last, thrust::less<>()); }
template <class D, class It>
It max_element(const system::cdna4::execution_policy<D>& exec, It first, It last) { return max_element(exec, first, last, thrust::less<>()); }
template <class D, class It>
pair<It, It> minmax_element(const system::cdna4::execution_policy<D>& exec, It first, It last) { return minmax_element(exec, first, last, thrust::less<>()); }
}}  // namespace system::cdna4
}  // namespace thrust
