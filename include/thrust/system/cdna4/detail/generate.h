// The cdna4 device system's generate (the counterpart of thrust/system/cuda/detail/generate.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/generate.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/generate.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class G>
void generate(const system::cdna4::execution_policy<D>& exec, It first, It last, G gen) {
  typedef typename thrust::detail::unwrap_iterator<It>::type Out;
  system::cdna4::detail::for_each_index(exec.derived(), (std::int64_t)(last - first),
                                        thrust::detail::generate_body<Out, G>{thrust::detail::unwrap(first), gen}, "generate: failed to synchronize");
}
}}  // namespace system::cdna4
}  // namespace thrust
