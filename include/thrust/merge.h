// thrust::merge / merge_by_key (thrust/merge.h): stable merge of two sorted ranges — of equivalent
// elements those of the first range come first (testing/merge.cu, merge_by_key.cu).  Device ranges
// run the merge-path kernels of system/cdna4/detail/merge_engine.h (compiled by hipcc); host ranges
// the sequential algorithm.
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>
#if defined(__HIPCC__)
#include <thrust/system/cdna4/detail/merge_engine.h>
#endif

#include <thrust/system/cdna4/detail/merge.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/merge.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In1, class In2, class Out, class Comp>
Out merge(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  return merge(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, last2, result, comp);
}
template <class D, class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>
pair<KOut, VOut> merge_by_key(const detail::execution_policy_base<D>& exec, K1 kfirst1, K1 klast1, K2 kfirst2, K2 klast2, V1 vfirst1, V2 vfirst2, KOut kresult, VOut vresult, Comp comp) {
  return merge_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst1, klast1, kfirst2, klast2, vfirst1, vfirst2, kresult, vresult, comp);
}
// ---- host
template <class In1, class In2, class Out, class Comp>
Out merge(const system::cpp::detail::par_t&, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  return std::merge(first1, last1, first2, last2, result, comp);
}
template <class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>
pair<KOut, VOut> merge_by_key(const system::cpp::detail::par_t&, K1 kfirst1, K1 klast1, K2 kfirst2, K2 klast2, V1 vfirst1, V2 vfirst2,
                              KOut kresult, VOut vresult, Comp comp) {
  // thrust/system/detail/sequential/merge.inl: take from the second range only when its key is strictly before
  while (kfirst1 != klast1 && kfirst2 != klast2) {
    if (comp(*kfirst2, *kfirst1)) { *kresult = *kfirst2; *vresult = *vfirst2; ++kfirst2; ++vfirst2; }
    else { *kresult = *kfirst1; *vresult = *vfirst1; ++kfirst1; ++vfirst1; }
    ++kresult; ++vresult;
  }
  for (; kfirst1 != klast1; ++kfirst1, ++vfirst1, ++kresult, ++vresult) { *kresult = *kfirst1; *vresult = *vfirst1; }
  for (; kfirst2 != klast2; ++kfirst2, ++vfirst2, ++kresult, ++vresult) { *kresult = *kfirst2; *vresult = *vfirst2; }
  return pair<KOut, VOut>(kresult, vresult);
}
// ---- default comparison, and the forms without a policy
namespace detail {
template <class Policy, class In1, class In2, class Out>
Out composed_merge(const Policy& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return merge(exec, f1, l1, f2, l2, r, less<typename detail::value_of<In1>::type>()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In1, class In2, class Out>
Out merge(execution_policy<D_>& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return thrust::detail::composed_merge(exec, f1, l1, f2, l2, r); }
}}  // namespace system::cdna4
template <class D_, class In1, class In2, class Out>
Out merge(const detail::execution_policy_base<D_>& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return merge(detail::derived_cast(detail::strip_const(exec)), f1, l1, f2, l2, r); }
template <class In1, class In2, class Out>
Out merge(const system::cpp::detail::par_t& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return detail::composed_merge(exec, f1, l1, f2, l2, r); }
template <class In1, class In2, class Out, class Comp, detail::enable_if_device<In1, In2, Out, Comp> = 0>
Out merge(In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp c) { return merge(typename detail::implicit_policy<In1, In2, Out, Comp>::type(), f1, l1, f2, l2, r, c); }
template <class In1, class In2, class Out, class Comp, detail::enable_if_host<In1, In2, Out, Comp> = 0>
Out merge(In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp c) { return merge(host, f1, l1, f2, l2, r, c); }
template <class In1, class In2, class Out, detail::enable_if_device<In1, In2, Out> = 0>
Out merge(In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return merge(typename detail::implicit_policy<In1, In2, Out>::type(), f1, l1, f2, l2, r); }
template <class In1, class In2, class Out, detail::enable_if_host<In1, In2, Out> = 0>
Out merge(In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return merge(host, f1, l1, f2, l2, r); }

namespace detail {
template <class Policy, class K1, class K2, class V1, class V2, class KOut, class VOut>
pair<KOut, VOut> composed_merge_by_key(const Policy& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) {
  return merge_by_key(exec, kf1, kl1, kf2, kl2, v1, v2, kr, vr, less<typename detail::value_of<K1>::type>());
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class K1, class K2, class V1, class V2, class KOut, class VOut>
pair<KOut, VOut> merge_by_key(execution_policy<D_>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return thrust::detail::composed_merge_by_key(exec, kf1, kl1, kf2, kl2, v1, v2, kr, vr); }
}}  // namespace system::cdna4
template <class D_, class K1, class K2, class V1, class V2, class KOut, class VOut>
pair<KOut, VOut> merge_by_key(const detail::execution_policy_base<D_>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return merge_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, v1, v2, kr, vr); }
template <class K1, class K2, class V1, class V2, class KOut, class VOut>
pair<KOut, VOut> merge_by_key(const system::cpp::detail::par_t& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return detail::composed_merge_by_key(exec, kf1, kl1, kf2, kl2, v1, v2, kr, vr); }
template <class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp, detail::enable_if_device<K1, K2, V1, V2, KOut, VOut, Comp> = 0>
pair<KOut, VOut> merge_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp c) { return merge_by_key(typename detail::implicit_policy<K1, K2, V1, V2, KOut, VOut, Comp>::type(), kf1, kl1, kf2, kl2, v1, v2, kr, vr, c); }
template <class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp, detail::enable_if_host<K1, K2, V1, V2, KOut, VOut, Comp> = 0>
pair<KOut, VOut> merge_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp c) { return merge_by_key(host, kf1, kl1, kf2, kl2, v1, v2, kr, vr, c); }
template <class K1, class K2, class V1, class V2, class KOut, class VOut, detail::enable_if_device<K1, K2, V1, V2, KOut, VOut> = 0>
pair<KOut, VOut> merge_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return merge_by_key(typename detail::implicit_policy<K1, K2, V1, V2, KOut, VOut>::type(), kf1, kl1, kf2, kl2, v1, v2, kr, vr); }
template <class K1, class K2, class V1, class V2, class KOut, class VOut, detail::enable_if_host<K1, K2, V1, V2, KOut, VOut> = 0>
pair<KOut, VOut> merge_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return merge_by_key(host, kf1, kl1, kf2, kl2, v1, v2, kr, vr); }
}  // namespace thrust
