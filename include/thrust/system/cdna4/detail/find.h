// The cdna4 device system's find (the counterpart of thrust/system/cuda/detail/find.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/find.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/find.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class Pred>
It find_if(const system::cdna4::execution_policy<D>& exec, It first, It last, Pred pred) { return thrust::detail::find_first<false>(exec.derived(), first, last, pred); }
template <class D, class It, class Pred>
It find_if_not(const system::cdna4::execution_policy<D>& exec, It first, It last, Pred pred) { return thrust::detail::find_first<true>(exec.derived(), first, last, pred); }
}}  // namespace system::cdna4
}  // namespace thrust
