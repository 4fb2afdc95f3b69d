// The algorithms of the hot path under thrust::seq: sort, stable_sort, sort_by_key,
// stable_sort_by_key, inclusive_scan, exclusive_scan, the by-key scans and reduce_by_key as
// __host__ __device__ loops in the calling thread.  Semantics: thrust/system/detail/sequential/
// sort.inl:42-200, scan.h:40-114, scan_by_key.h:46-142, reduce_by_key.h:43-95.  On the host they
// serve thrust::seq as they serve thrust::host; inside a kernel they are what a functor calls on
// a range that belongs to its thread (testing/cuda/sort.cu:18-105).
#pragma once
#include <cstdint>
#include <iterator>
#include <thrust/detail/seq.h>
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/detail/sequential/sort.h>

namespace thrust {

// ---- sort family -------------------------------------------------------------------
template <class It, class Compare>
THRUST_CDNA4_HD void stable_sort(const detail::seq_t&, It first, It last, Compare comp) {
  namespace sq = system::detail::sequential;
  sq::stable_sort_in_place(sq::keys_only<It>{first}, first, (std::int64_t)(last - first), comp);
}
template <class It>
THRUST_CDNA4_HD void stable_sort(const detail::seq_t& e, It first, It last) {
  stable_sort(e, first, last, less<typename std::iterator_traits<It>::value_type>());
}
template <class It, class Compare>
THRUST_CDNA4_HD void sort(const detail::seq_t& e, It first, It last, Compare comp) { stable_sort(e, first, last, comp); }
template <class It>
THRUST_CDNA4_HD void sort(const detail::seq_t& e, It first, It last) { stable_sort(e, first, last); }
template <class KIt, class VIt, class Compare>
THRUST_CDNA4_HD void stable_sort_by_key(const detail::seq_t&, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  namespace sq = system::detail::sequential;
  sq::stable_sort_in_place(sq::keys_and_values<KIt, VIt>{kfirst, vfirst}, kfirst, (std::int64_t)(klast - kfirst), comp);
}
template <class KIt, class VIt>
THRUST_CDNA4_HD void stable_sort_by_key(const detail::seq_t& e, KIt kfirst, KIt klast, VIt vfirst) {
  stable_sort_by_key(e, kfirst, klast, vfirst, less<typename std::iterator_traits<KIt>::value_type>());
}
template <class KIt, class VIt, class Compare>
THRUST_CDNA4_HD void sort_by_key(const detail::seq_t& e, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  stable_sort_by_key(e, kfirst, klast, vfirst, comp);
}
template <class KIt, class VIt>
THRUST_CDNA4_HD void sort_by_key(const detail::seq_t& e, KIt kfirst, KIt klast, VIt vfirst) { stable_sort_by_key(e, kfirst, klast, vfirst); }

// ---- scans: the accumulator is the input's value type (inclusive) or the type of the initial
//      value (exclusive), thrust/system/detail/sequential/scan.h:54-55, :91-92; an element is
//      read before its result is written, so a scan may run in place ------------------------
template <class InIt, class OutIt, class Op>
THRUST_CDNA4_HD OutIt inclusive_scan(const detail::seq_t&, InIt first, InIt last, OutIt result, Op op) {
  typedef typename std::iterator_traits<InIt>::value_type V;
  if (first != last) {
    V sum = *first;
    *result = sum;
    for (++first, ++result; first != last; ++first, ++result) {
      sum = op(sum, (V)*first);
      *result = sum;
    }
  }
  return result;
}
template <class InIt, class OutIt>
THRUST_CDNA4_HD OutIt inclusive_scan(const detail::seq_t& e, InIt first, InIt last, OutIt result) {
  return inclusive_scan(e, first, last, result, plus<>());
}
template <class InIt, class OutIt, class T, class Op>
THRUST_CDNA4_HD OutIt exclusive_scan(const detail::seq_t&, InIt first, InIt last, OutIt result, T init, Op op) {
  if (first != last) {
    T sum = init;
    for (; first != last; ++first, ++result) {
      const T x = *first;
      *result = sum;
      sum = op(sum, x);
    }
  }
  return result;
}
template <class InIt, class OutIt, class T>
THRUST_CDNA4_HD OutIt exclusive_scan(const detail::seq_t& e, InIt first, InIt last, OutIt result, T init) {
  return exclusive_scan(e, first, last, result, init, plus<>());
}
template <class InIt, class OutIt>
THRUST_CDNA4_HD OutIt exclusive_scan(const detail::seq_t& e, InIt first, InIt last, OutIt result) {
  return exclusive_scan(e, first, last, result, typename std::iterator_traits<InIt>::value_type(0), plus<>());
}

// ---- by-key scans (thrust/system/detail/sequential/scan_by_key.h:46-142): a key that differs
//      from its predecessor's starts a new segment ------------------------------------------
template <class KIt, class VIt, class OutIt, class Pred, class Op>
THRUST_CDNA4_HD OutIt inclusive_scan_by_key(const detail::seq_t&, KIt kfirst, KIt klast, VIt vfirst, OutIt result, Pred pred, Op op) {
  typedef typename std::iterator_traits<KIt>::value_type K;
  typedef typename std::iterator_traits<VIt>::value_type V;
  if (kfirst != klast) {
    K prev_key = *kfirst;
    V prev_value = *vfirst;
    *result = prev_value;
    for (++kfirst, ++vfirst, ++result; kfirst != klast; ++kfirst, ++vfirst, ++result) {
      const K key = *kfirst;
      if (pred(prev_key, key)) prev_value = op(prev_value, (V)*vfirst);
      else prev_value = *vfirst;
      *result = prev_value;
      prev_key = key;
    }
  }
  return result;
}
template <class KIt, class VIt, class OutIt, class Pred>
THRUST_CDNA4_HD OutIt inclusive_scan_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, OutIt r, Pred pred) {
  return inclusive_scan_by_key(e, kf, kl, vf, r, pred, plus<>());
}
template <class KIt, class VIt, class OutIt>
THRUST_CDNA4_HD OutIt inclusive_scan_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, OutIt r) {
  return inclusive_scan_by_key(e, kf, kl, vf, r, equal_to<>(), plus<>());
}
template <class KIt, class VIt, class OutIt, class T, class Pred, class Op>
THRUST_CDNA4_HD OutIt exclusive_scan_by_key(const detail::seq_t&, KIt kfirst, KIt klast, VIt vfirst, OutIt result, T init, Pred pred,
                                            Op op) {
  typedef typename std::iterator_traits<KIt>::value_type K;
  if (kfirst != klast) {
    K prev_key = *kfirst;
    T x = *vfirst;  // read before the result is written: the scan may run in place
    T next = init;
    *result = next;
    next = op(next, x);
    for (++kfirst, ++vfirst, ++result; kfirst != klast; ++kfirst, ++vfirst, ++result) {
      const K key = *kfirst;
      x = *vfirst;
      if (!pred(prev_key, key)) next = init;
      *result = next;
      next = op(next, x);
      prev_key = key;
    }
  }
  return result;
}
template <class KIt, class VIt, class OutIt, class T, class Pred>
THRUST_CDNA4_HD OutIt exclusive_scan_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, OutIt r, T init, Pred pred) {
  return exclusive_scan_by_key(e, kf, kl, vf, r, init, pred, plus<>());
}
template <class KIt, class VIt, class OutIt, class T>
THRUST_CDNA4_HD OutIt exclusive_scan_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, OutIt r, T init) {
  return exclusive_scan_by_key(e, kf, kl, vf, r, init, equal_to<>(), plus<>());
}
template <class KIt, class VIt, class OutIt>
THRUST_CDNA4_HD OutIt exclusive_scan_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, OutIt r) {
  return exclusive_scan_by_key(e, kf, kl, vf, r, typename std::iterator_traits<VIt>::value_type(0), equal_to<>(), plus<>());
}

// ---- reduce_by_key (thrust/system/detail/sequential/reduce_by_key.h:43-95) ------------------
template <class KIt, class VIt, class KOut, class VOut, class Pred, class Op>
THRUST_CDNA4_HD pair<KOut, VOut> reduce_by_key(const detail::seq_t&, KIt kfirst, KIt klast, VIt vfirst, KOut kout, VOut vout, Pred pred,
                                               Op op) {
  typedef typename std::iterator_traits<KIt>::value_type K;
  typedef typename std::iterator_traits<VIt>::value_type V;
  if (kfirst != klast) {
    K run_key = *kfirst;
    V run_value = *vfirst;
    for (++kfirst, ++vfirst; kfirst != klast; ++kfirst, ++vfirst) {
      const K key = *kfirst;
      const V value = *vfirst;
      if (pred(run_key, key)) {
        run_value = op(run_value, value);
      } else {
        *kout = run_key;
        *vout = run_value;
        ++kout;
        ++vout;
        run_key = key;
        run_value = value;
      }
    }
    *kout = run_key;
    *vout = run_value;
    ++kout;
    ++vout;
  }
  return pair<KOut, VOut>(kout, vout);
}
template <class KIt, class VIt, class KOut, class VOut, class Pred>
THRUST_CDNA4_HD pair<KOut, VOut> reduce_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred) {
  return reduce_by_key(e, kf, kl, vf, ko, vo, pred, plus<>());
}
template <class KIt, class VIt, class KOut, class VOut>
THRUST_CDNA4_HD pair<KOut, VOut> reduce_by_key(const detail::seq_t& e, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  return reduce_by_key(e, kf, kl, vf, ko, vo, equal_to<>(), plus<>());
}

}  // namespace thrust
