// The cdna4 device system's shuffle_copy (the counterpart of thrust/system/cuda/detail/shuffle_copy.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/shuffle.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/shuffle.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out, class URBG>
void shuffle_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out result, URBG&& g) {
  THRUST_CDNA4_NEEDS_HIPCC(In);
  const std::uint64_t m = (std::uint64_t)(last - first);
  if (m == 0) return;
  thrust::detail::feistel_bijection bijection(m, g);
#if defined(__HIPCC__)
  typedef typename thrust::detail::unwrap_iterator<In>::type RawIn;
  typedef typename thrust::detail::unwrap_iterator<Out>::type RawOut;
  system::cdna4::detail::generic::select(system::cdna4::detail::stream_of(exec.derived()), (std::int64_t)bijection.nearest_power_of_two(),
                                         thrust::detail::shuffle_op<RawIn, RawOut>{thrust::detail::unwrap(first), thrust::detail::unwrap(result), m, bijection});
#else
  (void)exec; (void)result;
#endif
}
}}  // namespace system::cdna4
}  // namespace thrust
