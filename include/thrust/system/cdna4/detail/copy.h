// The cdna4 device system's copy (the counterpart of thrust/system/cuda/detail/copy.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/copy.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/copy.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out>
Out copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out) {
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::transform_n(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(out), n, identity<typename thrust::detail::value_of<In>::type>());
  return out + n;
}
// contiguous device ranges of one type: a stream-ordered memcpy, no kernel template
template <class D, class T>
device_ptr<typename std::remove_const<T>::type> copy(const system::cdna4::execution_policy<D>& exec, device_ptr<T> first, device_ptr<T> last,
                                                     device_ptr<typename std::remove_const<T>::type> out) {
  namespace sd = system::cdna4::detail;
  const std::size_t n = (std::size_t)(last - first);
  if (n) sd::throw_on_error(thrust_cdna4_memcpy_dtod(out.get(), first.get(), n * sizeof(T), sd::stream_of(exec.derived())), "copy");
  sd::synchronize_optional(exec.derived(), "copy: failed to synchronize");
  return out + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
