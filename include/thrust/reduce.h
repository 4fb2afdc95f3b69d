// thrust::reduce (thrust/reduce.h:78-) and thrust::reduce_by_key (thrust/reduce.h:691-).
// reduce_by_key: device ranges go to the single-pass segmented-reduction kernel; host ranges run
// the sequential loop (thrust/system/detail/sequential/reduce_by_key.h:43-95).  reduce: device
// ranges go to the generic reduction kernel templates (a translation unit compiled by hipcc).
#pragma once
#include <numeric>
#include <thrust/detail/iterator_util.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/scan.h>
#include <thrust/system/cdna4/detail/algorithms.h>
#include <thrust/system/detail/sequential/algorithms.h>

#include <thrust/iterator/transform_iterator.h>
namespace thrust {

// ---- device
namespace detail {
template <class K, class V, class KIn, class VIn, class KOut, class VOut, class Pred, class Op> struct reduce_by_key_has_kernel {
  static constexpr bool value = system::cdna4::detail::dtype_of<K>::supported && system::cdna4::detail::dtype_of<V>::supported &&
                                builtin_equal_on<Pred, K>::value && builtin_op_on<Op, V>::value &&
                                raw_pointer_to<KIn, K>::value && raw_pointer_to<VIn, V>::value &&
                                raw_pointer_to<KOut, K>::value && raw_pointer_to<VOut, V>::value;
};
template <class K, class V, class Policy, class KIn, class VIn, class KOut, class VOut, class Pred, class Op>
std::int64_t reduce_by_key_dispatch(const Policy& exec, KIn keys, VIn vals, KOut ko, VOut vo, std::int64_t n, Pred pred, Op op, std::true_type) {
#if defined(__HIPCC__)
  if (n >= (std::int64_t(1) << 32))  // beyond the precompiled kernels' range
    return system::cdna4::detail::generic_reduce_by_key<V>(exec, keys, vals, ko, vo, n, pred, op);
#else
  (void)pred; (void)op;  // without the kernel templates such a call fails with the C ABI's error code
#endif
  return system::cdna4::detail::reduce_by_key(exec, static_cast<const K*>(keys), static_cast<const V*>(vals), ko, vo, n,
                                              typename rebind_op<Pred, K>::type(), typename rebind_op<Op, V>::type());
}
template <class K, class V, class Policy, class KIn, class VIn, class KOut, class VOut, class Pred, class Op>
std::int64_t reduce_by_key_dispatch(const Policy& exec, KIn keys, VIn vals, KOut ko, VOut vo, std::int64_t n, Pred pred, Op op, std::false_type) {
  return system::cdna4::detail::generic_reduce_by_key<V>(exec, keys, vals, ko, vo, n, pred, op);
}
}  // namespace detail

}  // namespace thrust
#include <thrust/system/cdna4/detail/reduce_by_key.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/reduce.inl:33-44, :112-130):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class KIt, class VIt, class KOut, class VOut, class Pred, class Op>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst, KOut kout, VOut vout, Pred pred, Op op) {
  return reduce_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, kout, vout, pred, op);
}
template <class D, class KIt, class VIt, class KOut, class VOut, class Pred>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred p) {
  return reduce_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo, p);
}
template <class D, class KIt, class VIt, class KOut, class VOut>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  return reduce_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo);
}

// ---- host
template <class KIt, class VIt, class KOut, class VOut, class Pred, class Op>
pair<KOut, VOut> reduce_by_key(const system::cpp::detail::par_t&, KIt kfirst, KIt klast, VIt vfirst, KOut kout,
                               VOut vout, Pred pred, Op op) {
  typedef typename detail::elem<KIt>::type K;
  typedef typename detail::elem<VIt>::type V;
  if (kfirst != klast) {
    K temp_key = *kfirst;
    V temp_value = *vfirst;
    for (++kfirst, ++vfirst; kfirst != klast; ++kfirst, ++vfirst) {
      K key = *kfirst;
      V value = *vfirst;
      if (pred(temp_key, key)) {
        temp_value = op(temp_value, value);
      } else {
        *kout = temp_key; *vout = temp_value;
        ++kout; ++vout;
        temp_key = key; temp_value = value;
      }
    }
    *kout = temp_key; *vout = temp_value;
    ++kout; ++vout;
  }
  return thrust::make_pair(kout, vout);
}
template <class KIt, class VIt, class KOut, class VOut, class Pred>
pair<KOut, VOut> reduce_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred p) {
  return reduce_by_key(e, kf, kl, vf, ko, vo, p, plus<typename detail::elem<VIt>::type>());
}
template <class KIt, class VIt, class KOut, class VOut>
pair<KOut, VOut> reduce_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  return reduce_by_key(e, kf, kl, vf, ko, vo, equal_to<typename detail::elem<KIt>::type>());
}

// ---- no policy
#define THRUST_CDNA4_RBK(SYS, COND)                                                                                 \
  template <class K, class V, class KO, class VO, COND<K> = 0>                                                       \
  pair<KO, VO> reduce_by_key(K kf, K kl, V vf, KO ko, VO vo) { return reduce_by_key(SYS, kf, kl, vf, ko, vo); }       \
  template <class K, class V, class KO, class VO, class P, COND<K> = 0>                                              \
  pair<KO, VO> reduce_by_key(K kf, K kl, V vf, KO ko, VO vo, P p) { return reduce_by_key(SYS, kf, kl, vf, ko, vo, p); } \
  template <class K, class V, class KO, class VO, class P, class O, COND<K> = 0>                                     \
  pair<KO, VO> reduce_by_key(K kf, K kl, V vf, KO ko, VO vo, P p, O o) { return reduce_by_key(SYS, kf, kl, vf, ko, vo, p, o); }
THRUST_CDNA4_RBK(typename detail::implicit_policy<K>::type(), detail::enable_if_device)
THRUST_CDNA4_RBK(host, detail::enable_if_host)
#undef THRUST_CDNA4_RBK


}  // namespace thrust
#include <thrust/system/cdna4/detail/reduce.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/reduce.inl:33-44, :112-130):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class T, class Op>
T reduce(const detail::execution_policy_base<D>& exec, It first, It last, T init, Op op) {
  return reduce(detail::derived_cast(detail::strip_const(exec)), first, last, init, op);
}
template <class D, class It, class T>
T reduce(const detail::execution_policy_base<D>& exec, It first, It last, T init) {
  return reduce(detail::derived_cast(detail::strip_const(exec)), first, last, init);
}
template <class D, class It>
typename detail::value_of<It>::type reduce(const detail::execution_policy_base<D>& exec, It first, It last) {
  return reduce(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <class It, class T, class Op>
T reduce(const system::cpp::detail::par_t&, It first, It last, T init, Op op) { return std::accumulate(first, last, init, op); }
template <class It, class T>
T reduce(const system::cpp::detail::par_t&, It first, It last, T init) { return std::accumulate(first, last, init); }
template <class It>
typename detail::value_of<It>::type reduce(const system::cpp::detail::par_t&, It first, It last) {
  typedef typename detail::value_of<It>::type V;
  return std::accumulate(first, last, V(0));
}
template <class It, detail::enable_if_device<It> = 0> typename detail::value_of<It>::type reduce(It f, It l) { return reduce(typename detail::implicit_policy<It>::type(), f, l); }
template <class It, detail::enable_if_host<It> = 0> typename detail::value_of<It>::type reduce(It f, It l) { return reduce(host, f, l); }
template <class It, class T, detail::enable_if_device<It, T> = 0> T reduce(It f, It l, T init) { return reduce(typename detail::implicit_policy<It>::type(), f, l, init); }
template <class It, class T, detail::enable_if_host<It, T> = 0> T reduce(It f, It l, T init) { return reduce(host, f, l, init); }
template <class It, class T, class Op, detail::enable_if_device<It, T, Op> = 0> T reduce(It f, It l, T init, Op op) { return reduce(typename detail::implicit_policy<It>::type(), f, l, init, op); }
template <class It, class T, class Op, detail::enable_if_host<It, T, Op> = 0> T reduce(It f, It l, T init, Op op) { return reduce(host, f, l, init, op); }

}  // namespace thrust
