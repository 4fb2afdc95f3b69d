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

namespace thrust {

// ---- device
template <class D, class KIt, class VIt, class KOut, class VOut, class Pred, class Op>
pair<KOut, VOut> reduce_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst,
                               KOut kout, VOut vout, Pred, Op) {
  namespace sd = system::cdna4::detail;
  typedef typename detail::elem<KIt>::type K;
  typedef typename detail::elem<VIt>::type V;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  sd::contiguous_input<K, typename detail::unwrap_iterator<KIt>::type> keys(exec.derived(), detail::unwrap(kfirst), n);
  sd::contiguous_input<V, typename detail::unwrap_iterator<VIt>::type> vals(exec.derived(), detail::unwrap(vfirst), n);
  sd::contiguous_output<K, typename detail::unwrap_iterator<KOut>::type> ko(exec.derived(), detail::unwrap(kout), n);
  sd::contiguous_output<V, typename detail::unwrap_iterator<VOut>::type> vo(exec.derived(), detail::unwrap(vout), n);
  const std::int64_t runs = sd::reduce_by_key(exec.derived(), keys.data(), vals.data(), ko.data(), vo.data(), n,
                                              typename detail::rebind_op<Pred, K>::type(), typename detail::rebind_op<Op, V>::type());
  ko.flush(exec.derived(), runs);
  vo.flush(exec.derived(), runs);
  return thrust::make_pair(kout + runs, vout + runs);
}
template <class D, class KIt, class VIt, class KOut, class VOut, class Pred>
pair<KOut, VOut> reduce_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred p) {
  return reduce_by_key(exec, kf, kl, vf, ko, vo, p, plus<typename detail::elem<VIt>::type>());
}
template <class D, class KIt, class VIt, class KOut, class VOut>
pair<KOut, VOut> reduce_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  return reduce_by_key(exec, kf, kl, vf, ko, vo, equal_to<typename detail::elem<KIt>::type>());
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
THRUST_CDNA4_RBK(device, detail::enable_if_device)
THRUST_CDNA4_RBK(host, detail::enable_if_host)
#undef THRUST_CDNA4_RBK


// ---------------------------------------------------------------------------------------
// reduce
// ---------------------------------------------------------------------------------------
template <class D, class It, class T, class Op>
T reduce(const system::cdna4::execution_policy<D>& exec, It first, It last, T init, Op op) {
  typedef typename detail::value_of<It>::type V;
  return system::cdna4::detail::transform_reduce_n(exec.derived(), detail::unwrap(first),
                                                   (std::int64_t)(last - first), identity<V>(), init, op);
}
template <class D, class It, class T>
T reduce(const system::cdna4::execution_policy<D>& exec, It first, It last, T init) { return reduce(exec, first, last, init, plus<T>()); }
template <class D, class It>
typename detail::value_of<It>::type reduce(const system::cdna4::execution_policy<D>& exec, It first, It last) {
  typedef typename detail::value_of<It>::type V;
  return reduce(exec, first, last, V(0), plus<V>());
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
template <class It, detail::enable_if_device<It> = 0> typename detail::value_of<It>::type reduce(It f, It l) { return reduce(device, f, l); }
template <class It, detail::enable_if_host<It> = 0> typename detail::value_of<It>::type reduce(It f, It l) { return reduce(host, f, l); }
template <class It, class T, detail::enable_if_device<It> = 0> T reduce(It f, It l, T init) { return reduce(device, f, l, init); }
template <class It, class T, detail::enable_if_host<It> = 0> T reduce(It f, It l, T init) { return reduce(host, f, l, init); }
template <class It, class T, class Op, detail::enable_if_device<It> = 0> T reduce(It f, It l, T init, Op op) { return reduce(device, f, l, init, op); }
template <class It, class T, class Op, detail::enable_if_host<It> = 0> T reduce(It f, It l, T init, Op op) { return reduce(host, f, l, init, op); }

}  // namespace thrust
