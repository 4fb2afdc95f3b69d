// The cdna4 device system's inner_product (the counterpart of thrust/system/cuda/detail/inner_product.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/inner_product.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/inner_product.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It1, class It2, class T, class Op1, class Op2>
T inner_product(const system::cdna4::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2) {
  return system::cdna4::detail::reduce_index(
      exec.derived(), (std::int64_t)(last1 - first1),
      thrust::detail::product_at<typename thrust::detail::unwrap_iterator<It1>::type, typename thrust::detail::unwrap_iterator<It2>::type, Op2, T>{
          thrust::detail::unwrap(first1), thrust::detail::unwrap(first2), op2},
      init, op1);
}
}}  // namespace system::cdna4
}  // namespace thrust
