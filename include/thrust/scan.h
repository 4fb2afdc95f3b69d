// thrust::inclusive_scan / exclusive_scan and the *_by_key forms (thrust/scan.h).
// Device ranges go to the single-pass look-back kernels; host ranges run the sequential
// loops (thrust/system/detail/sequential/scan.h:47-114, scan_by_key.h:46-142).
#pragma once
#include <iterator>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/algorithms.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust {

namespace detail {
template <class It>
struct elem {
  typedef typename std::remove_const<typename value_of<It>::type>::type type;
};
// functor re-bound to the element type, so thrust::plus<> and thrust::plus<int> select the same kernel
template <class Op, class T> struct rebind_op { typedef Op type; };
template <template <class> class F, class T> struct rebind_op<F<void>, T> { typedef F<T> type; };
}  // namespace detail

// ===================================================================== scan, device
template <class D, class InIt, class OutIt, class Op>
OutIt inclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result, Op) {
  namespace sd = system::cdna4::detail;
  typedef typename detail::elem<InIt>::type T;
  const std::int64_t n = (std::int64_t)(last - first);
  sd::contiguous_input<T, typename detail::unwrap_iterator<InIt>::type> in(exec.derived(), detail::unwrap(first), n);
  sd::contiguous_output<T, typename detail::unwrap_iterator<OutIt>::type> out(exec.derived(), detail::unwrap(result), n);
  sd::scan(exec.derived(), in.data(), out.data(), n, false, (const T*)nullptr, typename detail::rebind_op<Op, T>::type());
  out.flush(exec.derived(), n);
  return result + n;
}
template <class D, class InIt, class OutIt>
OutIt inclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result) {
  return inclusive_scan(exec, first, last, result, plus<typename detail::elem<InIt>::type>());
}
// The accumulator of an exclusive scan has the type of `init` (thrust/system/cuda/detail/scan.h:142-154);
// the kernels accumulate in the element type, so the two must be the same type.
template <class D, class InIt, class OutIt, class T, class Op>
OutIt exclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result, T init, Op) {
  namespace sd = system::cdna4::detail;
  typedef typename detail::elem<InIt>::type V;
  static_assert(std::is_same<V, T>::value,
                "cdna4 exclusive_scan: init must have the element type (it is the accumulator type)");
  const std::int64_t n = (std::int64_t)(last - first);
  sd::contiguous_input<V, typename detail::unwrap_iterator<InIt>::type> in(exec.derived(), detail::unwrap(first), n);
  sd::contiguous_output<V, typename detail::unwrap_iterator<OutIt>::type> out(exec.derived(), detail::unwrap(result), n);
  sd::scan(exec.derived(), in.data(), out.data(), n, true, &init, typename detail::rebind_op<Op, V>::type());
  out.flush(exec.derived(), n);
  return result + n;
}
template <class D, class InIt, class OutIt, class T>
OutIt exclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result, T init) {
  return exclusive_scan(exec, first, last, result, init, plus<typename detail::elem<InIt>::type>());
}
template <class D, class InIt, class OutIt>
OutIt exclusive_scan(const system::cdna4::execution_policy<D>& exec, InIt first, InIt last, OutIt result) {
  typedef typename detail::elem<InIt>::type V;
  return exclusive_scan(exec, first, last, result, V(), plus<V>());  // thrust/system/cuda/detail/scan.h:347-348
}

// ===================================================================== scan, host
template <class InIt, class OutIt, class Op>
OutIt inclusive_scan(const system::cpp::detail::par_t&, InIt first, InIt last, OutIt result, Op op) {
  typedef typename detail::elem<InIt>::type V;
  if (first != last) {
    V sum = *first;
    *result = sum;
    for (++first, ++result; first != last; ++first, ++result) *result = sum = op(sum, *first);
  }
  return result;
}
template <class InIt, class OutIt>
OutIt inclusive_scan(const system::cpp::detail::par_t& e, InIt first, InIt last, OutIt result) {
  return inclusive_scan(e, first, last, result, plus<typename detail::elem<InIt>::type>());
}
template <class InIt, class OutIt, class T, class Op>
OutIt exclusive_scan(const system::cpp::detail::par_t&, InIt first, InIt last, OutIt result, T init, Op op) {
  if (first != last) {
    T tmp = *first;
    T sum = init;
    *result = sum;
    sum = op(sum, tmp);
    for (++first, ++result; first != last; ++first, ++result) {
      tmp = *first;
      *result = sum;
      sum = op(sum, tmp);
    }
  }
  return result;
}
template <class InIt, class OutIt, class T>
OutIt exclusive_scan(const system::cpp::detail::par_t& e, InIt first, InIt last, OutIt result, T init) {
  return exclusive_scan(e, first, last, result, init, plus<T>());
}
template <class InIt, class OutIt>
OutIt exclusive_scan(const system::cpp::detail::par_t& e, InIt first, InIt last, OutIt result) {
  typedef typename detail::elem<InIt>::type V;
  return exclusive_scan(e, first, last, result, V(), plus<V>());
}

// ===================================================================== scan, no policy
template <class InIt, class OutIt, detail::enable_if_device<InIt> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r) { return inclusive_scan(device, f, l, r); }
template <class InIt, class OutIt, class Op, detail::enable_if_device<InIt> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r, Op op) { return inclusive_scan(device, f, l, r, op); }
template <class InIt, class OutIt, detail::enable_if_host<InIt> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r) { return inclusive_scan(host, f, l, r); }
template <class InIt, class OutIt, class Op, detail::enable_if_host<InIt> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r, Op op) { return inclusive_scan(host, f, l, r, op); }

template <class InIt, class OutIt, detail::enable_if_device<InIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r) { return exclusive_scan(device, f, l, r); }
template <class InIt, class OutIt, class T, detail::enable_if_device<InIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init) { return exclusive_scan(device, f, l, r, init); }
template <class InIt, class OutIt, class T, class Op, detail::enable_if_device<InIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init, Op op) { return exclusive_scan(device, f, l, r, init, op); }
template <class InIt, class OutIt, detail::enable_if_host<InIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r) { return exclusive_scan(host, f, l, r); }
template <class InIt, class OutIt, class T, detail::enable_if_host<InIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init) { return exclusive_scan(host, f, l, r, init); }
template <class InIt, class OutIt, class T, class Op, detail::enable_if_host<InIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init, Op op) { return exclusive_scan(host, f, l, r, init, op); }

// ===================================================================== scan_by_key, device
template <class D, class KIt, class VIt, class OutIt, class Pred, class Op>
OutIt inclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst,
                            OutIt result, Pred, Op) {
  namespace sd = system::cdna4::detail;
  typedef typename detail::elem<KIt>::type K;
  typedef typename detail::elem<VIt>::type V;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  sd::contiguous_input<K, typename detail::unwrap_iterator<KIt>::type> keys(exec.derived(), detail::unwrap(kfirst), n);
  sd::contiguous_input<V, typename detail::unwrap_iterator<VIt>::type> vals(exec.derived(), detail::unwrap(vfirst), n);
  sd::contiguous_output<V, typename detail::unwrap_iterator<OutIt>::type> out(exec.derived(), detail::unwrap(result), n);
  sd::scan_by_key(exec.derived(), keys.data(), vals.data(), out.data(), n, false, (const V*)nullptr,
                  typename detail::rebind_op<Pred, K>::type(), typename detail::rebind_op<Op, V>::type());
  out.flush(exec.derived(), n);
  return result + n;
}
template <class D, class KIt, class VIt, class OutIt, class Pred>
OutIt inclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, Pred p) {
  return inclusive_scan_by_key(exec, kf, kl, vf, r, p, plus<typename detail::elem<VIt>::type>());
}
template <class D, class KIt, class VIt, class OutIt>
OutIt inclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r) {
  return inclusive_scan_by_key(exec, kf, kl, vf, r, equal_to<typename detail::elem<KIt>::type>());
}
template <class D, class KIt, class VIt, class OutIt, class T, class Pred, class Op>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst,
                            OutIt result, T init, Pred, Op) {
  namespace sd = system::cdna4::detail;
  typedef typename detail::elem<KIt>::type K;
  typedef typename detail::elem<VIt>::type V;
  static_assert(std::is_same<V, T>::value, "cdna4 exclusive_scan_by_key: init must have the values' element type");
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  sd::contiguous_input<K, typename detail::unwrap_iterator<KIt>::type> keys(exec.derived(), detail::unwrap(kfirst), n);
  sd::contiguous_input<V, typename detail::unwrap_iterator<VIt>::type> vals(exec.derived(), detail::unwrap(vfirst), n);
  sd::contiguous_output<V, typename detail::unwrap_iterator<OutIt>::type> out(exec.derived(), detail::unwrap(result), n);
  sd::scan_by_key(exec.derived(), keys.data(), vals.data(), out.data(), n, true, &init,
                  typename detail::rebind_op<Pred, K>::type(), typename detail::rebind_op<Op, V>::type());
  out.flush(exec.derived(), n);
  return result + n;
}
template <class D, class KIt, class VIt, class OutIt, class T, class Pred>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, T init, Pred p) {
  return exclusive_scan_by_key(exec, kf, kl, vf, r, init, p, plus<typename detail::elem<VIt>::type>());
}
template <class D, class KIt, class VIt, class OutIt, class T>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, T init) {
  return exclusive_scan_by_key(exec, kf, kl, vf, r, init, equal_to<typename detail::elem<KIt>::type>());
}
template <class D, class KIt, class VIt, class OutIt>
OutIt exclusive_scan_by_key(const system::cdna4::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r) {
  return exclusive_scan_by_key(exec, kf, kl, vf, r, typename detail::elem<VIt>::type());
}

// ===================================================================== scan_by_key, host
template <class KIt, class VIt, class OutIt, class Pred, class Op>
OutIt inclusive_scan_by_key(const system::cpp::detail::par_t&, KIt kfirst, KIt klast, VIt vfirst, OutIt result,
                            Pred pred, Op op) {
  typedef typename detail::elem<KIt>::type K;
  typedef typename detail::elem<VIt>::type V;
  if (kfirst != klast) {
    K prev_key = *kfirst;
    V prev = *vfirst;
    *result = prev;
    for (++kfirst, ++vfirst, ++result; kfirst != klast; ++kfirst, ++vfirst, ++result) {
      K key = *kfirst;
      if (pred(prev_key, key)) *result = prev = op(prev, *vfirst);
      else *result = prev = *vfirst;
      prev_key = key;
    }
  }
  return result;
}
template <class KIt, class VIt, class OutIt, class Pred>
OutIt inclusive_scan_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, OutIt r, Pred p) {
  return inclusive_scan_by_key(e, kf, kl, vf, r, p, plus<typename detail::elem<VIt>::type>());
}
template <class KIt, class VIt, class OutIt>
OutIt inclusive_scan_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, OutIt r) {
  return inclusive_scan_by_key(e, kf, kl, vf, r, equal_to<typename detail::elem<KIt>::type>());
}
template <class KIt, class VIt, class OutIt, class T, class Pred, class Op>
OutIt exclusive_scan_by_key(const system::cpp::detail::par_t&, KIt kfirst, KIt klast, VIt vfirst, OutIt result,
                            T init, Pred pred, Op op) {
  typedef typename detail::elem<KIt>::type K;
  if (kfirst != klast) {
    K temp_key = *kfirst;
    T temp_value = *vfirst;
    T next = init;
    *result = next;
    next = op(next, temp_value);
    for (++kfirst, ++vfirst, ++result; kfirst != klast; ++kfirst, ++vfirst, ++result) {
      K key = *kfirst;
      temp_value = *vfirst;
      if (!pred(temp_key, key)) next = init;
      *result = next;
      next = op(next, temp_value);
      temp_key = key;
    }
  }
  return result;
}
template <class KIt, class VIt, class OutIt, class T, class Pred>
OutIt exclusive_scan_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, OutIt r, T init, Pred p) {
  return exclusive_scan_by_key(e, kf, kl, vf, r, init, p, plus<T>());
}
template <class KIt, class VIt, class OutIt, class T>
OutIt exclusive_scan_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, OutIt r, T init) {
  return exclusive_scan_by_key(e, kf, kl, vf, r, init, equal_to<typename detail::elem<KIt>::type>());
}
template <class KIt, class VIt, class OutIt>
OutIt exclusive_scan_by_key(const system::cpp::detail::par_t& e, KIt kf, KIt kl, VIt vf, OutIt r) {
  return exclusive_scan_by_key(e, kf, kl, vf, r, typename detail::elem<VIt>::type());
}

// ===================================================================== scan_by_key, no policy
#define THRUST_CDNA4_SBK(NAME, SYS, COND)                                                                          \
  template <class K, class V, class O, COND<K> = 0> O NAME(K kf, K kl, V vf, O r) { return NAME(SYS, kf, kl, vf, r); } \
  template <class K, class V, class O, class A, COND<K> = 0> O NAME(K kf, K kl, V vf, O r, A a) { return NAME(SYS, kf, kl, vf, r, a); } \
  template <class K, class V, class O, class A, class B, COND<K> = 0> O NAME(K kf, K kl, V vf, O r, A a, B b) { return NAME(SYS, kf, kl, vf, r, a, b); } \
  template <class K, class V, class O, class A, class B, class C, COND<K> = 0> O NAME(K kf, K kl, V vf, O r, A a, B b, C c) { return NAME(SYS, kf, kl, vf, r, a, b, c); }
THRUST_CDNA4_SBK(inclusive_scan_by_key, device, detail::enable_if_device)
THRUST_CDNA4_SBK(inclusive_scan_by_key, host, detail::enable_if_host)
THRUST_CDNA4_SBK(exclusive_scan_by_key, device, detail::enable_if_device)
THRUST_CDNA4_SBK(exclusive_scan_by_key, host, detail::enable_if_host)
#undef THRUST_CDNA4_SBK

}  // namespace thrust
