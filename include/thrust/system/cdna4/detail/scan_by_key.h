// The cdna4 device system's scan_by_key (the counterpart of thrust/system/cuda/detail/scan_by_key.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/scan.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/scan.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// The accumulator has the value input's type for the inclusive form and the type of `init` for
// the exclusive one (thrust/system/cuda/detail/scan_by_key.h:69-282).
template <class D, class KIt, class VIt, class OutIt, class Pred, class Op>
OutIt inclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst,
                            OutIt result, Pred pred, Op op) {
  typedef typename thrust::detail::elem<KIt>::type K;
  typedef typename thrust::detail::elem<VIt>::type V;
  typedef typename thrust::detail::unwrap_iterator<KIt>::type KIn;
  typedef typename thrust::detail::unwrap_iterator<VIt>::type VIn;
  typedef typename thrust::detail::unwrap_iterator<OutIt>::type Out;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  thrust::detail::scan_by_key_dispatch<false, K>(exec.derived(), thrust::detail::unwrap(kfirst), thrust::detail::unwrap(vfirst), thrust::detail::unwrap(result), n,
                                         V(), pred, op,
                                         std::integral_constant<bool, thrust::detail::scan_by_key_has_kernel<K, V, KIn, VIn, Out, Pred, Op>::value>());
  return result + n;
}
template <class D, class KIt, class VIt, class OutIt, class Pred>
OutIt inclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, Pred p) {
  return inclusive_scan_by_key(exec, kf, kl, vf, r, p, plus<>());
}
template <class D, class KIt, class VIt, class OutIt>
OutIt inclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r) {
  return inclusive_scan_by_key(exec, kf, kl, vf, r, equal_to<>());
}
template <class D, class KIt, class VIt, class OutIt, class T, class Pred, class Op>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst,
                            OutIt result, T init, Pred pred, Op op) {
  typedef typename thrust::detail::elem<KIt>::type K;
  typedef typename thrust::detail::unwrap_iterator<KIt>::type KIn;
  typedef typename thrust::detail::unwrap_iterator<VIt>::type VIn;
  typedef typename thrust::detail::unwrap_iterator<OutIt>::type Out;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  thrust::detail::scan_by_key_dispatch<true, K>(exec.derived(), thrust::detail::unwrap(kfirst), thrust::detail::unwrap(vfirst), thrust::detail::unwrap(result), n,
                                        init, pred, op,
                                        std::integral_constant<bool, thrust::detail::scan_by_key_has_kernel<K, T, KIn, VIn, Out, Pred, Op>::value>());
  return result + n;
}
template <class D, class KIt, class VIt, class OutIt, class T, class Pred>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, T init, Pred p) {
  return exclusive_scan_by_key(exec, kf, kl, vf, r, init, p, plus<>());
}
template <class D, class KIt, class VIt, class OutIt, class T>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, T init) {
  return exclusive_scan_by_key(exec, kf, kl, vf, r, init, equal_to<>());
}
template <class D, class KIt, class VIt, class OutIt>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r) {
  return exclusive_scan_by_key(exec, kf, kl, vf, r, typename thrust::detail::elem<VIt>::type());
}
}}  // namespace system::cdna4
}  // namespace thrust
