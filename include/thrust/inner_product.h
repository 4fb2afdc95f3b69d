// thrust::inner_product (thrust/inner_product.h): init (+) a[0](*)b[0] (+) a[1](*)b[1] ...
#pragma once
#include <numeric>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

#include <thrust/reduce.h>
namespace thrust {
namespace detail {
template <class A, class B, class Op2, class T> struct product_at {
  A a; B b; mutable Op2 op2;
  THRUST_CDNA4_HD T operator()(std::int64_t i) const { return (T)op2(a[i], b[i]); }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/inner_product.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/inner_product.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It1, class It2, class T, class Op1, class Op2>
T inner_product(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2) {
  return inner_product(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, init, op1, op2);
}
template <class It1, class It2, class T, class Op1, class Op2>
T inner_product(const system::cpp::detail::par_t&, It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2) {
  return std::inner_product(first1, last1, first2, init, op1, op2);
}
namespace detail {
template <class Policy, class It1, class It2, class T>
T composed_inner_product(const Policy& exec, It1 f1, It1 l1, It2 f2, T init) { return inner_product(exec, f1, l1, f2, init, plus<T>(), multiplies<T>()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It1, class It2, class T>
T inner_product(execution_policy<D_>& exec, It1 f1, It1 l1, It2 f2, T init) { return thrust::detail::composed_inner_product(exec, f1, l1, f2, init); }
}}  // namespace system::cdna4
template <class D_, class It1, class It2, class T>
T inner_product(const detail::execution_policy_base<D_>& exec, It1 f1, It1 l1, It2 f2, T init) { return inner_product(detail::derived_cast(detail::strip_const(exec)), f1, l1, f2, init); }
template <class It1, class It2, class T>
T inner_product(const system::cpp::detail::par_t& exec, It1 f1, It1 l1, It2 f2, T init) { return detail::composed_inner_product(exec, f1, l1, f2, init); }
template <class It1, class It2, class T, detail::enable_if_device<It1, It2, T> = 0> T inner_product(It1 f1, It1 l1, It2 f2, T init) { return inner_product(typename detail::implicit_policy<It1, It2, T>::type(), f1, l1, f2, init); }
template <class It1, class It2, class T, detail::enable_if_host<It1, It2, T> = 0> T inner_product(It1 f1, It1 l1, It2 f2, T init) { return inner_product(host, f1, l1, f2, init); }
template <class It1, class It2, class T, class O1, class O2, detail::enable_if_device<It1, It2, T, O1, O2> = 0>
T inner_product(It1 f1, It1 l1, It2 f2, T init, O1 o1, O2 o2) { return inner_product(typename detail::implicit_policy<It1, It2, T, O1, O2>::type(), f1, l1, f2, init, o1, o2); }
template <class It1, class It2, class T, class O1, class O2, detail::enable_if_host<It1, It2, T, O1, O2> = 0>
T inner_product(It1 f1, It1 l1, It2 f2, T init, O1 o1, O2 o2) { return inner_product(host, f1, l1, f2, init, o1, o2); }
}  // namespace thrust
