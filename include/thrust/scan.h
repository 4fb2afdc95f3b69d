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
#include <thrust/system/cdna4/detail/scan_generic.h>
#include <thrust/system/detail/sequential/algorithms.h>

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
namespace detail {
// The precompiled kernels serve raw device pointers to one arithmetic type under one of the four
// built-in operators of that type (or its transparent form); everything else goes to the kernel
// templates of scan_generic.h.
template <class Op, class T> struct builtin_op_on { static constexpr bool value = false; };
template <template <class> class F, class T> struct builtin_op_on<F<T>, T> {
  static constexpr bool value = system::cdna4::detail::op_code<F<T>>::value >= 0;
};
template <template <class> class F, class T> struct builtin_op_on<F<void>, T> {
  static constexpr bool value = system::cdna4::detail::op_code<F<T>>::value >= 0;
};
template <class P, class T> struct raw_pointer_to {
  static constexpr bool value = std::is_pointer<P>::value &&
      std::is_same<typename std::remove_cv<typename std::remove_pointer<P>::type>::type, T>::value;
};
template <class T, class In, class Out, class Op> struct scan_has_kernel {
  static constexpr bool value = system::cdna4::detail::dtype_of<T>::supported && builtin_op_on<Op, T>::value &&
                                raw_pointer_to<In, T>::value && raw_pointer_to<Out, T>::value;
};

template <bool EXCLUSIVE, class Policy, class T, class In, class Out, class Op>
void scan_dispatch(const Policy& exec, In in, Out out, std::int64_t n, T init, Op, std::true_type) {
  system::cdna4::detail::scan(exec, static_cast<const T*>(in), out, n, EXCLUSIVE, EXCLUSIVE ? &init : (const T*)nullptr,
                              typename rebind_op<Op, T>::type());
}
template <bool EXCLUSIVE, class Policy, class T, class In, class Out, class Op>
void scan_dispatch(const Policy& exec, In in, Out out, std::int64_t n, T init, Op op, std::false_type) {
  system::cdna4::detail::generic_scan<EXCLUSIVE, T>(exec, in, out, n, init, op);
}
}  // namespace detail

}  // namespace thrust
#include <thrust/system/cdna4/detail/scan.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/scan.inl:35-48):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class InIt, class OutIt, class Op>
OutIt inclusive_scan(const detail::execution_policy_base<D>& exec, InIt first, InIt last, OutIt result, Op op) {
  return inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, op);
}
template <class D, class InIt, class OutIt>
OutIt inclusive_scan(const detail::execution_policy_base<D>& exec, InIt first, InIt last, OutIt result) {
  return inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <class D, class InIt, class OutIt, class T, class Op>
OutIt exclusive_scan(const detail::execution_policy_base<D>& exec, InIt first, InIt last, OutIt result, T init, Op op) {
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, init, op);
}
template <class D, class InIt, class OutIt, class T>
OutIt exclusive_scan(const detail::execution_policy_base<D>& exec, InIt first, InIt last, OutIt result, T init) {
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, init);
}
template <class D, class InIt, class OutIt>
OutIt exclusive_scan(const detail::execution_policy_base<D>& exec, InIt first, InIt last, OutIt result) {
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result);
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
template <class InIt, class OutIt, detail::enable_if_device<InIt, OutIt> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r) { return inclusive_scan(typename detail::implicit_policy<InIt>::type(), f, l, r); }
template <class InIt, class OutIt, class Op, detail::enable_if_device<InIt, OutIt, Op> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r, Op op) { return inclusive_scan(typename detail::implicit_policy<InIt>::type(), f, l, r, op); }
template <class InIt, class OutIt, detail::enable_if_host<InIt, OutIt> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r) { return inclusive_scan(host, f, l, r); }
template <class InIt, class OutIt, class Op, detail::enable_if_host<InIt, OutIt, Op> = 0>
OutIt inclusive_scan(InIt f, InIt l, OutIt r, Op op) { return inclusive_scan(host, f, l, r, op); }

template <class InIt, class OutIt, detail::enable_if_device<InIt, OutIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r) { return exclusive_scan(typename detail::implicit_policy<InIt>::type(), f, l, r); }
template <class InIt, class OutIt, class T, detail::enable_if_device<InIt, OutIt, T> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init) { return exclusive_scan(typename detail::implicit_policy<InIt>::type(), f, l, r, init); }
template <class InIt, class OutIt, class T, class Op, detail::enable_if_device<InIt, OutIt, T, Op> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init, Op op) { return exclusive_scan(typename detail::implicit_policy<InIt>::type(), f, l, r, init, op); }
template <class InIt, class OutIt, detail::enable_if_host<InIt, OutIt> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r) { return exclusive_scan(host, f, l, r); }
template <class InIt, class OutIt, class T, detail::enable_if_host<InIt, OutIt, T> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init) { return exclusive_scan(host, f, l, r, init); }
template <class InIt, class OutIt, class T, class Op, detail::enable_if_host<InIt, OutIt, T, Op> = 0>
OutIt exclusive_scan(InIt f, InIt l, OutIt r, T init, Op op) { return exclusive_scan(host, f, l, r, init, op); }

// ===================================================================== scan_by_key, device
namespace detail {
template <class Pred, class K> struct builtin_equal_on { static constexpr bool value = false; };
template <class K> struct builtin_equal_on<equal_to<K>, K> { static constexpr bool value = true; };
template <class K> struct builtin_equal_on<equal_to<void>, K> { static constexpr bool value = true; };
template <class K, class V, class KIn, class VIn, class Out, class Pred, class Op> struct scan_by_key_has_kernel {
  static constexpr bool value = system::cdna4::detail::dtype_of<K>::supported && system::cdna4::detail::dtype_of<V>::supported &&
                                builtin_equal_on<Pred, K>::value && builtin_op_on<Op, V>::value &&
                                raw_pointer_to<KIn, K>::value && raw_pointer_to<VIn, V>::value && raw_pointer_to<Out, V>::value;
};
template <bool EXCLUSIVE, class K, class Policy, class V, class KIn, class VIn, class Out, class Pred, class Op>
void scan_by_key_dispatch(const Policy& exec, KIn keys, VIn vals, Out out, std::int64_t n, V init, Pred pred, Op op, std::true_type) {
#if defined(__HIPCC__)
  if (n >= (std::int64_t(1) << 32)) {  // beyond the precompiled kernels' range
    system::cdna4::detail::generic_scan_by_key<EXCLUSIVE, V>(exec, keys, vals, out, n, init, pred, op);
    return;
  }
#else
  (void)pred; (void)op;  // without the kernel templates such a call fails with the C ABI's error code
#endif
  system::cdna4::detail::scan_by_key(exec, static_cast<const K*>(keys), static_cast<const V*>(vals), out, n, EXCLUSIVE,
                                     EXCLUSIVE ? &init : (const V*)nullptr, typename rebind_op<Pred, K>::type(),
                                     typename rebind_op<Op, V>::type());
}
template <bool EXCLUSIVE, class K, class Policy, class V, class KIn, class VIn, class Out, class Pred, class Op>
void scan_by_key_dispatch(const Policy& exec, KIn keys, VIn vals, Out out, std::int64_t n, V init, Pred pred, Op op, std::false_type) {
  system::cdna4::detail::generic_scan_by_key<EXCLUSIVE, V>(exec, keys, vals, out, n, init, pred, op);
}
}  // namespace detail

}  // namespace thrust
#include <thrust/system/cdna4/detail/scan_by_key.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/scan.inl:35-48):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class KIt, class VIt, class OutIt, class Pred, class Op>
OutIt inclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst, OutIt result, Pred pred, Op op) {
  return inclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, result, pred, op);
}
template <class D, class KIt, class VIt, class OutIt, class Pred>
OutIt inclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, Pred p) {
  return inclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, r, p);
}
template <class D, class KIt, class VIt, class OutIt>
OutIt inclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r) {
  return inclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, r);
}
template <class D, class KIt, class VIt, class OutIt, class T, class Pred, class Op>
OutIt exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kfirst, KIt klast, VIt vfirst, OutIt result, T init, Pred pred, Op op) {
  return exclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, result, init, pred, op);
}
template <class D, class KIt, class VIt, class OutIt, class T, class Pred>
OutIt exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, T init, Pred p) {
  return exclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, r, init, p);
}
template <class D, class KIt, class VIt, class OutIt, class T>
OutIt exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r, T init) {
  return exclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, r, init);
}
template <class D, class KIt, class VIt, class OutIt>
OutIt exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, OutIt r) {
  return exclusive_scan_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, r);
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
THRUST_CDNA4_SBK(inclusive_scan_by_key, typename detail::implicit_policy<K>::type(), detail::enable_if_device)
THRUST_CDNA4_SBK(inclusive_scan_by_key, host, detail::enable_if_host)
THRUST_CDNA4_SBK(exclusive_scan_by_key, typename detail::implicit_policy<K>::type(), detail::enable_if_device)
THRUST_CDNA4_SBK(exclusive_scan_by_key, host, detail::enable_if_host)
#undef THRUST_CDNA4_SBK

}  // namespace thrust
