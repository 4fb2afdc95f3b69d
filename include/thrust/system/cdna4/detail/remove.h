// The cdna4 device system's remove (the counterpart of thrust/system/cuda/detail/remove.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/remove.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/remove.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
namespace detail {
template <class Policy, class In, class Pred>
In remove_if_in_place(const Policy& exec, In first, In last, Pred pred, std::true_type /* contiguous */) {
  typedef typename thrust::detail::value_of<In>::type V;
  const std::int64_t n = (std::int64_t)(last - first);
  scratch_copy<V> tmp((const V*)thrust::detail::unwrap(first), n, stream_of(exec));
  return first + copy_flagged_n<true>(exec, tmp.data(), thrust::detail::unwrap(first), n, pred);
}
// a range that is no array (a zip of arrays, say): its elements are gathered into a temporary first
template <class Policy, class In, class Pred>
In remove_if_in_place(const Policy& exec, In first, In last, Pred pred, std::false_type) {
  typedef typename thrust::detail::value_of<In>::type V;
  const std::int64_t n = (std::int64_t)(last - first);
  temporary_storage buf((std::size_t)n * sizeof(V), exec);
  V* tmp = static_cast<V*>(buf.data());
  thrust::copy(exec, first, last, thrust::device_ptr<V>(tmp));
  return first + copy_flagged_n<true>(exec, (const V*)tmp, thrust::detail::unwrap(first), n, pred);
}
}  // namespace detail
template <class D, class In, class Out, class Pred>
Out remove_copy_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out, Pred pred) {
  return out + system::cdna4::detail::copy_flagged_n<true>(exec.derived(), detail::as_input(thrust::detail::unwrap(first)), thrust::detail::unwrap(out),
                                                           (std::int64_t)(last - first), pred);
}
template <class D, class In, class Pred>
In remove_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Pred pred) {
  return detail::remove_if_in_place(exec.derived(), first, last, pred, std::is_pointer<typename thrust::detail::unwrap_iterator<In>::type>());
}
}}  // namespace system::cdna4
}  // namespace thrust
