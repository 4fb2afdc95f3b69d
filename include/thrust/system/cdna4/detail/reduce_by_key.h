// The cdna4 device system's reduce_by_key (the counterpart of thrust/system/cuda/detail/reduce_by_key.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/reduce.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/reduce.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// Raw device pointers to arithmetic types under equal_to and a built-in operator run the
// precompiled segmented-reduction kernel; everything else (user predicates and operators, fancy
// iterators read in place, more than 2^32 - 1 elements) the kernel templates of scan_generic.h.
template <class D, class KIt, class VIt, class KOut, class VOut, class Pred, class Op>
pair<KOut, VOut> reduce_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst,
                               KOut kout, VOut vout, Pred pred, Op op) {
  typedef typename thrust::detail::elem<KIt>::type K;
  typedef typename thrust::detail::elem<VIt>::type V;
  typedef typename thrust::detail::unwrap_iterator<KIt>::type KIn;
  typedef typename thrust::detail::unwrap_iterator<VIt>::type VIn;
  typedef typename thrust::detail::unwrap_iterator<KOut>::type KO;
  typedef typename thrust::detail::unwrap_iterator<VOut>::type VO;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  const std::int64_t runs = thrust::detail::reduce_by_key_dispatch<K, V>(
      exec.derived(), thrust::detail::unwrap(kfirst), thrust::detail::unwrap(vfirst), thrust::detail::unwrap(kout), thrust::detail::unwrap(vout), n, pred, op,
      std::integral_constant<bool, thrust::detail::reduce_by_key_has_kernel<K, V, KIn, VIn, KO, VO, Pred, Op>::value>());
  return thrust::make_pair(kout + runs, vout + runs);
}
template <class D, class KIt, class VIt, class KOut, class VOut, class Pred>
pair<KOut, VOut> reduce_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred p) {
  return reduce_by_key(exec, kf, kl, vf, ko, vo, p, plus<>());
}
template <class D, class KIt, class VIt, class KOut, class VOut>
pair<KOut, VOut> reduce_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  return reduce_by_key(exec, kf, kl, vf, ko, vo, equal_to<>());
}
}}  // namespace system::cdna4
}  // namespace thrust
