// The cdna4 device system's fill (the counterpart of thrust/system/cuda/detail/fill.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/fill.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/fill.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class V>
void fill(const system::cdna4::execution_policy<D>& exec, It first, It last, const V& value) {
  thrust::detail::fill_device(exec.derived(), first, (std::int64_t)(last - first), value);
}
}}  // namespace system::cdna4
}  // namespace thrust
