// The cdna4 device system's adjacent_difference (the counterpart of thrust/system/cuda/detail/adjacent_difference.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/adjacent_difference.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/adjacent_difference.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out, class Op>
Out adjacent_difference(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out, Op op) {
  namespace sd = system::cdna4::detail;
  typedef typename thrust::detail::value_of<In>::type V;
  const std::int64_t n = (std::int64_t)(last - first);
  if (n <= 0) return out;
  auto in = thrust::detail::unwrap(first);
  auto o = thrust::detail::unwrap(out);
  if (thrust::detail::same_address(in, o)) {
    sd::scratch_copy<V> tmp((const V*)(const void*)sd::address_of(in), n, sd::stream_of(exec.derived()));
    sd::adjacent_difference_n(exec.derived(), tmp.data(), o, n, op);
    // the temporary goes back to the pool in stream order, after the kernel that reads it
  } else {
    sd::adjacent_difference_n(exec.derived(), in, o, n, op);
  }
  return out + n;
}
}}  // namespace system::cdna4
}  // namespace thrust
