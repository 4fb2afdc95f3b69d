// The cdna4 device system's shuffle (the counterpart of thrust/system/cuda/detail/shuffle.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/shuffle.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/shuffle.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// in place: shuffle a copy back into the range
template <class D, class It, class URBG>
void shuffle(const system::cdna4::execution_policy<D>& exec, It first, It last, URBG&& g) {
  typedef typename std::iterator_traits<It>::value_type T;
  thrust::device_vector<T> copy(first, last);
  shuffle_copy(exec, copy.begin(), copy.end(), first, g);
}
}}  // namespace system::cdna4
}  // namespace thrust
