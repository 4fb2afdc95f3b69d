// The cdna4 device system's uninitialized_copy (the counterpart of thrust/system/cuda/detail/uninitialized_copy.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/uninitialized_copy.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/uninitialized_copy.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class In, class Out>
Out uninitialized_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out result) { return copy(exec, first, last, result); }
}}  // namespace system::cdna4
}  // namespace thrust
