// The cdna4 device system's merge (the counterpart of thrust/system/cuda/detail/merge.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/merge.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/merge.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// ---- device
template <class D, class In1, class In2, class Out, class Comp>
Out merge(const system::cdna4::execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  THRUST_CDNA4_NEEDS_HIPCC(Comp);
  const std::int64_t na = (std::int64_t)(last1 - first1), nb = (std::int64_t)(last2 - first2);
#if defined(__HIPCC__)
  namespace m = system::cdna4::detail::merge2;
  m::merge<false>(system::cdna4::detail::stream_of(exec.derived()), thrust::detail::unwrap(first1), na, thrust::detail::unwrap(first2), nb, system::cdna4::detail::no_values(),
                  system::cdna4::detail::no_values(), thrust::detail::unwrap(result), system::cdna4::detail::no_values(), comp);
  system::cdna4::detail::synchronize_optional(exec.derived(), "merge: failed to synchronize");
#endif
  return result + (na + nb);
}
template <class D, class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>
pair<KOut, VOut> merge_by_key(const system::cdna4::execution_policy<D>& exec, K1 kfirst1, K1 klast1, K2 kfirst2, K2 klast2, V1 vfirst1,
                              V2 vfirst2, KOut kresult, VOut vresult, Comp comp) {
  THRUST_CDNA4_NEEDS_HIPCC(Comp);
  const std::int64_t na = (std::int64_t)(klast1 - kfirst1), nb = (std::int64_t)(klast2 - kfirst2);
#if defined(__HIPCC__)
  namespace m = system::cdna4::detail::merge2;
  m::merge<true>(system::cdna4::detail::stream_of(exec.derived()), thrust::detail::unwrap(kfirst1), na, thrust::detail::unwrap(kfirst2), nb,
                 thrust::detail::unwrap(vfirst1), thrust::detail::unwrap(vfirst2), thrust::detail::unwrap(kresult), thrust::detail::unwrap(vresult), comp);
  system::cdna4::detail::synchronize_optional(exec.derived(), "merge_by_key: failed to synchronize");
#else
  (void)vfirst1; (void)vfirst2;
#endif
  return pair<KOut, VOut>(kresult + (na + nb), vresult + (na + nb));
}
}}  // namespace system::cdna4
}  // namespace thrust
