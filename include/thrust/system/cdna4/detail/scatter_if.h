// The cdna4 device system's scatter_if (the counterpart of thrust/system/cuda/detail/scatter_if.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/scatter.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/scatter.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Map, class S, class Out, class Pred>
void scatter_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Map map, S stencil, Out output, Pred pred) {
  system::cdna4::detail::for_each_index(
      exec.derived(), (std::int64_t)(last - first),
      thrust::detail::scatter_if_body<typename thrust::detail::unwrap_iterator<In>::type, typename thrust::detail::unwrap_iterator<Map>::type,
                              typename thrust::detail::unwrap_iterator<S>::type, typename thrust::detail::unwrap_iterator<Out>::type, Pred>{
          thrust::detail::unwrap(first), thrust::detail::unwrap(map), thrust::detail::unwrap(stencil), thrust::detail::unwrap(output), pred},
      "scatter_if: failed to synchronize");
}
}}  // namespace system::cdna4
}  // namespace thrust
