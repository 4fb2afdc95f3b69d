// The cdna4 device system's gather_if (the counterpart of thrust/system/cuda/detail/gather_if.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/gather.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/gather.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class Map, class S, class In, class Out, class Pred>
Out gather_if(const system::cdna4::execution_policy<D>& exec, Map map_first, Map map_last, S stencil, In input, Out result, Pred pred) {
  const std::int64_t n = (std::int64_t)(map_last - map_first);
  system::cdna4::detail::for_each_index(
      exec.derived(), n,
      thrust::detail::gather_if_body<typename thrust::detail::unwrap_iterator<Map>::type, typename thrust::detail::unwrap_iterator<S>::type,
                             typename thrust::detail::unwrap_iterator<In>::type, typename thrust::detail::unwrap_iterator<Out>::type, Pred>{
          thrust::detail::unwrap(map_first), thrust::detail::unwrap(stencil), thrust::detail::unwrap(input), thrust::detail::unwrap(result), pred},
      "gather_if: failed to synchronize");
  return result + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
