// The cdna4 device system's remove (the counterpart of thrust/system/cuda/detail/remove.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/remove.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/remove.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out, class Pred>
Out remove_copy_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out, Pred pred) {
  typedef typename thrust::detail::value_of<In>::type V;
  const V* in = thrust::detail::unwrap(first);
  return out + system::cdna4::detail::copy_flagged_n<true>(exec.derived(), in, thrust::detail::unwrap(out), (std::int64_t)(last - first), pred);
}
template <class D, class In, class Pred>
In remove_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Pred pred) {
  typedef typename thrust::detail::value_of<In>::type V;
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::scratch_copy<V> tmp((const V*)thrust::detail::unwrap(first), n, system::cdna4::detail::stream_of(exec.derived()));
  return first + system::cdna4::detail::copy_flagged_n<true>(exec.derived(), tmp.data(), thrust::detail::unwrap(first), n, pred);
}
}}  // namespace system::cdna4
}  // namespace thrust
