// The cdna4 device system's copy_if (the counterpart of thrust/system/cuda/detail/copy_if.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/copy.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/copy.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out, class Pred>
Out copy_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out, Pred pred) {
  return out + system::cdna4::detail::copy_flagged_n<false>(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(out), (std::int64_t)(last - first), pred);
}
template <class D, class In, class St, class Out, class Pred>
Out copy_if(const system::cdna4::execution_policy<D>& exec, In first, In last, St stencil, Out out, Pred pred) {
  return out + system::cdna4::detail::copy_flagged_n<false>(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(stencil),
                                                            thrust::detail::unwrap(out), (std::int64_t)(last - first), pred);
}
}}  // namespace system::cdna4
}  // namespace thrust
