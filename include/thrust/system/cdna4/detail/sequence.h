// The cdna4 device system's sequence (the counterpart of thrust/system/cuda/detail/sequence.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/sequence.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/sequence.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class T>
void sequence(const system::cdna4::execution_policy<D>& exec, It first, It last, T init, T step) {
  // computed in the type of init and step, converted where it is stored
  // (thrust/system/detail/generic/sequence.inl:36-90)
  system::cdna4::detail::sequence_n(exec.derived(), thrust::detail::unwrap(first), (std::int64_t)(last - first), init, step);
}
template <class D, class It, class T>
void sequence(const system::cdna4::execution_policy<D>& exec, It first, It last, T init) { sequence(exec, first, last, init, T(1)); }
template <class D, class It, class = typename std::iterator_traits<It>::iterator_category>
void sequence(const system::cdna4::execution_policy<D>& exec, It first, It last) {
  typedef typename thrust::detail::value_of<It>::type V;
  sequence(exec, first, last, V(0), V(1));
}
}}  // namespace system::cdna4
}  // namespace thrust
