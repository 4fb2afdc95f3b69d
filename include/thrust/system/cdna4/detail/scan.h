// The cdna4 device system's scan (the counterpart of thrust/system/cuda/detail/scan.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/scan.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/scan.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// The accumulator of an inclusive scan has the input's value type (thrust/system/cuda/detail/scan.h:63).
template <class D, class InIt, class OutIt, class Op>
OutIt inclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result, Op op) {
  typedef typename thrust::detail::elem<InIt>::type T;
  typedef typename thrust::detail::unwrap_iterator<InIt>::type In;
  typedef typename thrust::detail::unwrap_iterator<OutIt>::type Out;
  const std::int64_t n = (std::int64_t)(last - first);
  thrust::detail::scan_dispatch<false>(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(result), n, T(), op,
                               std::integral_constant<bool, thrust::detail::scan_has_kernel<T, In, Out, Op>::value>());
  return result + n;
}
template <class D, class InIt, class OutIt>
OutIt inclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result) {
  return inclusive_scan(exec, first, last, result, plus<>());
}
// The accumulator of an exclusive scan has the type of `init` (thrust/system/cuda/detail/scan.h:142-154).
template <class D, class InIt, class OutIt, class T, class Op>
OutIt exclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result, T init, Op op) {
  typedef typename thrust::detail::unwrap_iterator<InIt>::type In;
  typedef typename thrust::detail::unwrap_iterator<OutIt>::type Out;
  const std::int64_t n = (std::int64_t)(last - first);
  thrust::detail::scan_dispatch<true>(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(result), n, init, op,
                              std::integral_constant<bool, thrust::detail::scan_has_kernel<T, In, Out, Op>::value>());
  return result + n;
}
template <class D, class InIt, class OutIt, class T>
OutIt exclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result, T init) {
  return exclusive_scan(exec, first, last, result, init, plus<>());
}
template <class D, class InIt, class OutIt>
OutIt exclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result) {
  typedef typename thrust::detail::elem<InIt>::type V;
  return exclusive_scan(exec, first, last, result, V(), plus<>());  // thrust/system/cuda/detail/scan.h:347-348
}
}}  // namespace system::cdna4
}  // namespace thrust
