// The cdna4 device system's transform (the counterpart of thrust/system/cuda/detail/transform.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/transform.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/transform.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out, class F>
Out transform(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out, F f) {
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::transform_n(exec.derived(), thrust::detail::unwrap(first),
                                     thrust::detail::unwrap(out), n, f);
  return out + n;
}
template <class D, class In1, class In2, class Out, class F>
Out transform(const system::cdna4::execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, Out out, F f) {
  const std::int64_t n = (std::int64_t)(last1 - first1);
  system::cdna4::detail::transform_n(exec.derived(), thrust::detail::unwrap(first1),
                                     thrust::detail::unwrap(first2), thrust::detail::unwrap(out), n, f);
  return out + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
