// thrust::set_difference / set_intersection / set_symmetric_difference / set_union and their
// _by_key forms (thrust/set_operations.h) on sorted ranges, with the multiset semantics of the
// sequential algorithms: an element found m times in the first range and n times in the second
// appears max(m - n, 0) / min(m, n) / |m - n| / max(m, n) times, elements (and values) of the first
// range first (testing/set_difference.cu, set_intersection.cu, set_symmetric_difference.cu,
// set_union.cu and their _by_key files).  Device ranges: one stable compaction per input range by
// a per-element rule, then a stable merge where two ranges contribute
// (system/cdna4/detail/merge_engine.h, compiled by hipcc).  Host ranges: the sequential loops.
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

namespace thrust {
namespace detail {
enum { set_difference_mode = 0, set_intersection_mode = 1, set_symmetric_difference_mode = 2, set_union_mode = 3 };
typedef system::cdna4::detail::no_values no_value_iterator;  // "no values" in the shared implementations

// ---- device: keys only (HAS_VALUES false; the value arguments are ignored) or keys with values
template <int MODE, bool HAS_VALUES, class D, class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>
std::int64_t set_operation(const system::cdna4::execution_policy<D>& exec, K1 kfirst1, K1 klast1, K2 kfirst2, K2 klast2, V1 vfirst1, V2 vfirst2,
                           KOut kresult, VOut vresult, Comp comp) {
  THRUST_CDNA4_NEEDS_HIPCC(Comp);
#if defined(__HIPCC__)
  namespace m = system::cdna4::detail::merge2;
  typedef typename std::iterator_traits<K1>::value_type KT1;
  typedef typename std::iterator_traits<K2>::value_type KT2;
  void* stream = system::cdna4::detail::stream_of(exec.derived());
  const std::int64_t na = (std::int64_t)(klast1 - kfirst1), nb = (std::int64_t)(klast2 - kfirst2);
  const auto a = unwrap(kfirst1);
  const auto b = unwrap(kfirst2);
  const auto va1 = unwrap(vfirst1);
  const auto vb2 = unwrap(vfirst2);
  const auto ko = unwrap(kresult);
  const auto vo = unwrap(vresult);
  std::int64_t count = 0;
  if (MODE == set_difference_mode) {
    count = m::set_select<false, HAS_VALUES>(stream, a, na, b, nb, va1, ko, vo, comp);
  } else if (MODE == set_intersection_mode) {
    count = m::set_select<true, HAS_VALUES>(stream, a, na, b, nb, va1, ko, vo, comp);
  } else {
    // what the second range adds: its elements that the first does not match
    typedef typename std::conditional<HAS_VALUES, typename std::iterator_traits<typename std::conditional<HAS_VALUES, V2, K2>::type>::value_type, char>::type VT2;
    system::cdna4::detail::temporary_storage tkb((std::size_t)(nb ? nb : 1) * sizeof(KT2), stream);
    system::cdna4::detail::temporary_storage tvb(HAS_VALUES ? (std::size_t)(nb ? nb : 1) * sizeof(VT2) : 0, stream);
    KT2* kb = static_cast<KT2*>(tkb.data());
    VT2* vb = static_cast<VT2*>(tvb.data());
    const std::int64_t cb = m::set_select<false, HAS_VALUES>(stream, b, nb, a, na, vb2, kb, vb, comp);
    if (MODE == set_union_mode) {
      m::merge<HAS_VALUES>(stream, a, na, kb, cb, va1, vb, ko, vo, comp);
      count = na + cb;
    } else {
      typedef typename std::conditional<HAS_VALUES, typename std::iterator_traits<typename std::conditional<HAS_VALUES, V1, K1>::type>::value_type, char>::type VT1;
      system::cdna4::detail::temporary_storage tka((std::size_t)(na ? na : 1) * sizeof(KT1), stream);
      system::cdna4::detail::temporary_storage tva(HAS_VALUES ? (std::size_t)(na ? na : 1) * sizeof(VT1) : 0, stream);
      KT1* ka = static_cast<KT1*>(tka.data());
      VT1* va = static_cast<VT1*>(tva.data());
      const std::int64_t ca = m::set_select<false, HAS_VALUES>(stream, a, na, b, nb, va1, ka, va, comp);
      m::merge<HAS_VALUES>(stream, ka, ca, kb, cb, va, vb, ko, vo, comp);
      count = ca + cb;
    }
    // the temporaries go back to the pool in stream order behind the merge
  }
  system::cdna4::detail::synchronize_optional(exec.derived(), "set operation: failed to synchronize");
  return count;
#else
  (void)exec; (void)kfirst1; (void)klast1; (void)kfirst2; (void)klast2; (void)vfirst1; (void)vfirst2; (void)kresult; (void)vresult; (void)comp;
  return 0;
#endif
}

// ---- host: the sequential loops (thrust/system/detail/sequential/set_operations.h), values along
template <bool HAS_VALUES> struct set_emit {
  template <class K, class V, class KOut, class VOut> static void put(K k, V v, KOut& ko, VOut& vo) { *ko = *k; *vo = *v; ++ko; ++vo; }
  template <class V> static void next(V& v) { ++v; }
};
template <> struct set_emit<false> {
  template <class K, class V, class KOut, class VOut> static void put(K k, V, KOut& ko, VOut&) { *ko = *k; ++ko; }
  template <class V> static void next(V&) {}
};
template <int MODE, bool HAS_VALUES, class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>
std::int64_t set_operation(const system::cpp::detail::par_t&, K1 k1, K1 l1, K2 k2, K2 l2, V1 v1, V2 v2, KOut ko, VOut vo, Comp comp) {
  typedef set_emit<HAS_VALUES> E;
  const KOut start = ko;
  while (k1 != l1 && k2 != l2) {
    if (comp(*k1, *k2)) {  // only in the first range
      if (MODE != set_intersection_mode) E::put(k1, v1, ko, vo);
      ++k1; E::next(v1);
    } else if (comp(*k2, *k1)) {  // only in the second
      if (MODE == set_symmetric_difference_mode || MODE == set_union_mode) E::put(k2, v2, ko, vo);
      ++k2; E::next(v2);
    } else {  // a matched pair
      if (MODE == set_intersection_mode || MODE == set_union_mode) E::put(k1, v1, ko, vo);
      ++k1; E::next(v1);
      ++k2; E::next(v2);
    }
  }
  if (MODE != set_intersection_mode)
    for (; k1 != l1; ++k1, E::next(v1)) E::put(k1, v1, ko, vo);
  if (MODE == set_symmetric_difference_mode || MODE == set_union_mode)
    for (; k2 != l2; ++k2, E::next(v2)) E::put(k2, v2, ko, vo);
  return (std::int64_t)(ko - start);
}
}  // namespace detail

// The four algorithms on keys: NAME(policy, first1, last1, first2, last2, result[, comp]) and the forms without a policy.
// The forms with a policy dispatch on the policy's own type by an unqualified call (thrust/detail/set_operations.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
#define THRUST_CDNA4_SET_OPERATION(NAME, MODE)                                                                                        \
  namespace system { namespace cdna4 {                                                                                               \
  template <class D, class In1, class In2, class Out, class Comp>                                                                     \
  Out NAME(execution_policy<D>& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp comp) {                                             \
    return r + thrust::detail::set_operation<MODE, false>(exec.derived(), f1, l1, f2, l2, thrust::detail::no_value_iterator(),        \
                                                          thrust::detail::no_value_iterator(), r, thrust::detail::no_value_iterator(), comp); \
  }                                                                                                                                   \
  template <class D, class In1, class In2, class Out>                                                                                 \
  Out NAME(execution_policy<D>& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) {                                                        \
    return NAME(exec, f1, l1, f2, l2, r, thrust::less<typename thrust::detail::value_of<In1>::type>());                               \
  }                                                                                                                                   \
  }}                                                                                                                                  \
  template <class D, class In1, class In2, class Out, class Comp>                                                                     \
  Out NAME(const detail::execution_policy_base<D>& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp comp) {                          \
    return NAME(detail::derived_cast(detail::strip_const(exec)), f1, l1, f2, l2, r, comp);                                            \
  }                                                                                                                                   \
  template <class D, class In1, class In2, class Out>                                                                                 \
  Out NAME(const detail::execution_policy_base<D>& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) {                                     \
    return NAME(detail::derived_cast(detail::strip_const(exec)), f1, l1, f2, l2, r);                                                  \
  }                                                                                                                                   \
  template <class In1, class In2, class Out, class Comp>                                                                              \
  Out NAME(const system::cpp::detail::par_t& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp comp) {                                \
    return r + detail::set_operation<MODE, false>(exec, f1, l1, f2, l2, detail::no_value_iterator(), detail::no_value_iterator(), r, \
                                                  detail::no_value_iterator(), comp);                                               \
  }                                                                                                                                   \
  template <class In1, class In2, class Out>                                                                                          \
  Out NAME(const system::cpp::detail::par_t& exec, In1 f1, In1 l1, In2 f2, In2 l2, Out r) {                                           \
    return NAME(exec, f1, l1, f2, l2, r, less<typename detail::value_of<In1>::type>());                                               \
  }                                                                                                                                   \
  template <class In1, class In2, class Out, class Comp, detail::enable_if_device<In1, In2, Out, Comp> = 0>                                           \
  Out NAME(In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp c) { return NAME(typename detail::implicit_policy<In1, In2, Out, Comp>::type(), f1, l1, f2, l2, r, c); }                              \
  template <class In1, class In2, class Out, class Comp, detail::enable_if_host<In1, In2, Out, Comp> = 0>                                             \
  Out NAME(In1 f1, In1 l1, In2 f2, In2 l2, Out r, Comp c) { return NAME(host, f1, l1, f2, l2, r, c); }                                \
  template <class In1, class In2, class Out, detail::enable_if_device<In1, In2, Out> = 0>                                                       \
  Out NAME(In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return NAME(typename detail::implicit_policy<In1, In2, Out>::type(), f1, l1, f2, l2, r); }                                         \
  template <class In1, class In2, class Out, detail::enable_if_host<In1, In2, Out> = 0>                                                         \
  Out NAME(In1 f1, In1 l1, In2 f2, In2 l2, Out r) { return NAME(host, f1, l1, f2, l2, r); }
THRUST_CDNA4_SET_OPERATION(set_difference, thrust::detail::set_difference_mode)
THRUST_CDNA4_SET_OPERATION(set_intersection, thrust::detail::set_intersection_mode)
THRUST_CDNA4_SET_OPERATION(set_symmetric_difference, thrust::detail::set_symmetric_difference_mode)
THRUST_CDNA4_SET_OPERATION(set_union, thrust::detail::set_union_mode)
#undef THRUST_CDNA4_SET_OPERATION

// The by-key forms with values for both ranges:
// NAME(policy, kfirst1, klast1, kfirst2, klast2, vfirst1, vfirst2, kresult, vresult[, comp]).
#define THRUST_CDNA4_SET_OPERATION_BY_KEY(NAME, MODE)                                                                                 \
  namespace system { namespace cdna4 {                                                                                               \
  template <class D, class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>                                      \
  pair<KOut, VOut> NAME(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp comp) {       \
    const std::int64_t c = thrust::detail::set_operation<MODE, true>(exec.derived(), kf1, kl1, kf2, kl2, v1, v2, kr, vr, comp);       \
    return pair<KOut, VOut>(kr + c, vr + c);                                                                                          \
  }                                                                                                                                   \
  template <class D, class K1, class K2, class V1, class V2, class KOut, class VOut>                                                  \
  pair<KOut, VOut> NAME(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) {                  \
    return NAME(exec, kf1, kl1, kf2, kl2, v1, v2, kr, vr, thrust::less<typename thrust::detail::value_of<K1>::type>());               \
  }                                                                                                                                   \
  }}                                                                                                                                  \
  template <class D, class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>                                      \
  pair<KOut, VOut> NAME(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp comp) { \
    return NAME(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, v1, v2, kr, vr, comp);                           \
  }                                                                                                                                   \
  template <class D, class K1, class K2, class V1, class V2, class KOut, class VOut>                                                  \
  pair<KOut, VOut> NAME(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { \
    return NAME(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, v1, v2, kr, vr);                                 \
  }                                                                                                                                   \
  template <class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp>                                               \
  pair<KOut, VOut> NAME(const system::cpp::detail::par_t& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp comp) { \
    const std::int64_t c = detail::set_operation<MODE, true>(exec, kf1, kl1, kf2, kl2, v1, v2, kr, vr, comp);                         \
    return pair<KOut, VOut>(kr + c, vr + c);                                                                                          \
  }                                                                                                                                   \
  template <class K1, class K2, class V1, class V2, class KOut, class VOut>                                                           \
  pair<KOut, VOut> NAME(const system::cpp::detail::par_t& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) {     \
    return NAME(exec, kf1, kl1, kf2, kl2, v1, v2, kr, vr, less<typename detail::value_of<K1>::type>());                               \
  }                                                                                                                                   \
  template <class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp, detail::enable_if_device<K1, K2, V1, V2, KOut, VOut, Comp> = 0>             \
  pair<KOut, VOut> NAME(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp c) { return NAME(typename detail::implicit_policy<K1, K2, V1, V2, KOut, VOut, Comp>::type(), kf1, kl1, kf2, kl2, v1, v2, kr, vr, c); } \
  template <class K1, class K2, class V1, class V2, class KOut, class VOut, class Comp, detail::enable_if_host<K1, K2, V1, V2, KOut, VOut, Comp> = 0>               \
  pair<KOut, VOut> NAME(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr, Comp c) { return NAME(host, kf1, kl1, kf2, kl2, v1, v2, kr, vr, c); } \
  template <class K1, class K2, class V1, class V2, class KOut, class VOut, detail::enable_if_device<K1, K2, V1, V2, KOut, VOut> = 0>                         \
  pair<KOut, VOut> NAME(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return NAME(typename detail::implicit_policy<K1, K2, V1, V2, KOut, VOut>::type(), kf1, kl1, kf2, kl2, v1, v2, kr, vr); } \
  template <class K1, class K2, class V1, class V2, class KOut, class VOut, detail::enable_if_host<K1, K2, V1, V2, KOut, VOut> = 0>                           \
  pair<KOut, VOut> NAME(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, V2 v2, KOut kr, VOut vr) { return NAME(host, kf1, kl1, kf2, kl2, v1, v2, kr, vr); }
THRUST_CDNA4_SET_OPERATION_BY_KEY(set_difference_by_key, thrust::detail::set_difference_mode)
THRUST_CDNA4_SET_OPERATION_BY_KEY(set_symmetric_difference_by_key, thrust::detail::set_symmetric_difference_mode)
THRUST_CDNA4_SET_OPERATION_BY_KEY(set_union_by_key, thrust::detail::set_union_mode)
#undef THRUST_CDNA4_SET_OPERATION_BY_KEY

// set_intersection_by_key takes values for the first range only (every result comes from it).
namespace system { namespace cdna4 {
template <class D, class K1, class K2, class V1, class KOut, class VOut, class Comp>
pair<KOut, VOut> set_intersection_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr, Comp comp) {
  const std::int64_t c = thrust::detail::set_operation<thrust::detail::set_intersection_mode, true>(exec.derived(), kf1, kl1, kf2, kl2, v1, v1, kr, vr, comp);
  return pair<KOut, VOut>(kr + c, vr + c);
}
template <class D, class K1, class K2, class V1, class KOut, class VOut>
pair<KOut, VOut> set_intersection_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr) {
  return set_intersection_by_key(exec, kf1, kl1, kf2, kl2, v1, kr, vr, thrust::less<typename thrust::detail::value_of<K1>::type>());
}
}}  // namespace system::cdna4
template <class D, class K1, class K2, class V1, class KOut, class VOut, class Comp>
pair<KOut, VOut> set_intersection_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr, Comp comp) {
  return set_intersection_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, v1, kr, vr, comp);
}
template <class D, class K1, class K2, class V1, class KOut, class VOut>
pair<KOut, VOut> set_intersection_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr) {
  return set_intersection_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, v1, kr, vr);
}
template <class K1, class K2, class V1, class KOut, class VOut, class Comp>
pair<KOut, VOut> set_intersection_by_key(const system::cpp::detail::par_t& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr, Comp comp) {
  const std::int64_t c = detail::set_operation<detail::set_intersection_mode, true>(exec, kf1, kl1, kf2, kl2, v1, v1, kr, vr, comp);
  return pair<KOut, VOut>(kr + c, vr + c);
}
template <class K1, class K2, class V1, class KOut, class VOut>
pair<KOut, VOut> set_intersection_by_key(const system::cpp::detail::par_t& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr) {
  return set_intersection_by_key(exec, kf1, kl1, kf2, kl2, v1, kr, vr, less<typename detail::value_of<K1>::type>());
}
template <class K1, class K2, class V1, class KOut, class VOut, class Comp, detail::enable_if_device<K1, K2, V1, KOut, VOut, Comp> = 0>
pair<KOut, VOut> set_intersection_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr, Comp c) { return set_intersection_by_key(typename detail::implicit_policy<K1, K2, V1, KOut, VOut, Comp>::type(), kf1, kl1, kf2, kl2, v1, kr, vr, c); }
template <class K1, class K2, class V1, class KOut, class VOut, class Comp, detail::enable_if_host<K1, K2, V1, KOut, VOut, Comp> = 0>
pair<KOut, VOut> set_intersection_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr, Comp c) { return set_intersection_by_key(host, kf1, kl1, kf2, kl2, v1, kr, vr, c); }
template <class K1, class K2, class V1, class KOut, class VOut, detail::enable_if_device<K1, K2, V1, KOut, VOut> = 0>
pair<KOut, VOut> set_intersection_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr) { return set_intersection_by_key(typename detail::implicit_policy<K1, K2, V1, KOut, VOut>::type(), kf1, kl1, kf2, kl2, v1, kr, vr); }
template <class K1, class K2, class V1, class KOut, class VOut, detail::enable_if_host<K1, K2, V1, KOut, VOut> = 0>
pair<KOut, VOut> set_intersection_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 v1, KOut kr, VOut vr) { return set_intersection_by_key(host, kf1, kl1, kf2, kl2, v1, kr, vr); }
}  // namespace thrust
