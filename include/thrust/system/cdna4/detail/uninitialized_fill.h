// The cdna4 device system's uninitialized_fill (the counterpart of thrust/system/cuda/detail/uninitialized_fill.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/uninitialized_fill.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/uninitialized_fill.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class T>
void uninitialized_fill(const system::cdna4::execution_policy<D>& exec, It first, It last, const T& x) { fill(exec, first, last, x); }
}}  // namespace system::cdna4
}  // namespace thrust
