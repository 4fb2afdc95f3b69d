// thrust::transform, unary and binary (thrust/transform.h; thrust/system/cuda/detail/transform.h).
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/for_each.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/system/cdna4/detail/transform.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/transform.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class F>
Out transform(const detail::execution_policy_base<D>& exec, In first, In last, Out out, F f) {
  return transform(detail::derived_cast(detail::strip_const(exec)), first, last, out, f);
}
template <class D, class In1, class In2, class Out, class F>
Out transform(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, Out out, F f) {
  return transform(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, out, f);
}
template <class In, class Out, class F>
Out transform(const system::cpp::detail::par_t&, In first, In last, Out out, F f) { return std::transform(first, last, out, f); }
template <class In1, class In2, class Out, class F>
Out transform(const system::cpp::detail::par_t&, In1 first1, In1 last1, In2 first2, Out out, F f) {
  return std::transform(first1, last1, first2, out, f);
}

template <class In, class Out, class F, detail::enable_if_device<In, Out, F> = 0>
Out transform(In f, In l, Out o, F fn) { return transform(typename detail::implicit_policy<In, Out, F>::type(), f, l, o, fn); }
template <class In, class Out, class F, detail::enable_if_host<In, Out, F> = 0>
Out transform(In f, In l, Out o, F fn) { return transform(host, f, l, o, fn); }
template <class In1, class In2, class Out, class F, detail::enable_if_device<In1, In2, Out, F> = 0,
          class = typename std::iterator_traits<In2>::iterator_category>
Out transform(In1 f, In1 l, In2 f2, Out o, F fn) { return transform(typename detail::implicit_policy<In1, In2, Out, F>::type(), f, l, f2, o, fn); }
template <class In1, class In2, class Out, class F, detail::enable_if_host<In1, In2, Out, F> = 0,
          class = typename std::iterator_traits<In2>::iterator_category>
Out transform(In1 f, In1 l, In2 f2, Out o, F fn) { return transform(host, f, l, f2, o, fn); }

// ---- transform_if (thrust/transform.h:316-724): result[i] = op(...) where the predicate holds on
//      the element (or on stencil[i]); the other positions of result are left as they are
namespace detail {
template <class In1, class In2, class St, class Out, class Op, class Pred, int ARITY, bool STENCIL>
struct transform_if_at {
  In1 a; In2 b; St stencil; Out out; Op op; Pred pred;
  template <class Index>
  THRUST_CDNA4_HD void operator()(Index i) {
    if (STENCIL ? (bool)pred(stencil[i]) : (bool)pred(a[i])) out[i] = apply(i, std::integral_constant<int, ARITY>());
  }
  template <class Index> THRUST_CDNA4_HD auto apply(Index i, std::integral_constant<int, 1>) -> decltype(op(a[i])) { return op(a[i]); }
  template <class Index> THRUST_CDNA4_HD auto apply(Index i, std::integral_constant<int, 2>) -> decltype(op(a[i], b[i])) { return op(a[i], b[i]); }
};
template <int ARITY, bool STENCIL, class Policy, class In1, class In2, class St, class Out, class Op, class Pred>
Out transform_if_n(const Policy& exec, In1 a, In2 b, St stencil, Out out, std::int64_t n, Op op, Pred pred) {
  typedef transform_if_at<typename unwrap_iterator<In1>::type, typename unwrap_iterator<In2>::type, typename unwrap_iterator<St>::type,
                          typename unwrap_iterator<Out>::type, Op, Pred, ARITY, STENCIL> F;
  thrust::for_each_n(exec, counting_iterator<std::int64_t>(0), n, F{unwrap(a), unwrap(b), unwrap(stencil), unwrap(out), op, pred});
  return out + n;
}
}  // namespace detail
namespace detail {
template <class Policy, class In, class Out, class Op, class Pred>
Out composed_transform_if(const Policy& exec, In first, In last, Out result, Op op, Pred pred) {
  return detail::transform_if_n<1, false>(exec, first, first, first, result, (std::int64_t)(last - first), op, pred);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out, class Op, class Pred>
Out transform_if(execution_policy<D_>& exec, In first, In last, Out result, Op op, Pred pred) { return thrust::detail::composed_transform_if(exec, first, last, result, op, pred); }
}}  // namespace system::cdna4
template <class D_, class In, class Out, class Op, class Pred>
Out transform_if(const detail::execution_policy_base<D_>& exec, In first, In last, Out result, Op op, Pred pred) { return transform_if(detail::derived_cast(detail::strip_const(exec)), first, last, result, op, pred); }
template <class In, class Out, class Op, class Pred>
Out transform_if(const system::cpp::detail::par_t& exec, In first, In last, Out result, Op op, Pred pred) { return detail::composed_transform_if(exec, first, last, result, op, pred); }
namespace detail {
template <class Policy, class In, class St, class Out, class Op, class Pred>
Out composed_transform_if(const Policy& exec, In first, In last, St stencil, Out result, Op op, Pred pred) {
  return detail::transform_if_n<1, true>(exec, first, first, stencil, result, (std::int64_t)(last - first), op, pred);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class St, class Out, class Op, class Pred>
Out transform_if(execution_policy<D_>& exec, In first, In last, St stencil, Out result, Op op, Pred pred) { return thrust::detail::composed_transform_if(exec, first, last, stencil, result, op, pred); }
}}  // namespace system::cdna4
template <class D_, class In, class St, class Out, class Op, class Pred>
Out transform_if(const detail::execution_policy_base<D_>& exec, In first, In last, St stencil, Out result, Op op, Pred pred) { return transform_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, result, op, pred); }
template <class In, class St, class Out, class Op, class Pred>
Out transform_if(const system::cpp::detail::par_t& exec, In first, In last, St stencil, Out result, Op op, Pred pred) { return detail::composed_transform_if(exec, first, last, stencil, result, op, pred); }
namespace detail {
template <class Policy, class In1, class In2, class St, class Out, class Op, class Pred>
Out composed_transform_if(const Policy& exec, In1 first1, In1 last1, In2 first2, St stencil, Out result, Op op, Pred pred) {
  return detail::transform_if_n<2, true>(exec, first1, first2, stencil, result, (std::int64_t)(last1 - first1), op, pred);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In1, class In2, class St, class Out, class Op, class Pred>
Out transform_if(execution_policy<D_>& exec, In1 first1, In1 last1, In2 first2, St stencil, Out result, Op op, Pred pred) { return thrust::detail::composed_transform_if(exec, first1, last1, first2, stencil, result, op, pred); }
}}  // namespace system::cdna4
template <class D_, class In1, class In2, class St, class Out, class Op, class Pred>
Out transform_if(const detail::execution_policy_base<D_>& exec, In1 first1, In1 last1, In2 first2, St stencil, Out result, Op op, Pred pred) { return transform_if(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, stencil, result, op, pred); }
template <class In1, class In2, class St, class Out, class Op, class Pred>
Out transform_if(const system::cpp::detail::par_t& exec, In1 first1, In1 last1, In2 first2, St stencil, Out result, Op op, Pred pred) { return detail::composed_transform_if(exec, first1, last1, first2, stencil, result, op, pred); }
#define THRUST_CDNA4_TRANSFORM_IF_NO_POLICY(SYS, COND)                                                                         \
  template <class In, class Out, class Op, class Pred, COND<In, Out, Op, Pred> = 0>                                                           \
  Out transform_if(In first, In last, Out result, Op op, Pred pred) { return transform_if(SYS(In, Out, Op, Pred), first, last, result, op, pred); } \
  template <class In, class St, class Out, class Op, class Pred, COND<In, St, Out, Op, Pred> = 0>                                                 \
  Out transform_if(In first, In last, St stencil, Out result, Op op, Pred pred) {                                              \
    return transform_if(SYS(In, St, Out, Op, Pred), first, last, stencil, result, op, pred);                                                          \
  }                                                                                                                            \
  template <class In1, class In2, class St, class Out, class Op, class Pred, COND<In1, In2, St, Out, Op, Pred> = 0>                                    \
  Out transform_if(In1 first1, In1 last1, In2 first2, St stencil, Out result, Op op, Pred pred) {                              \
    return transform_if(SYS(In1, In2, St, Out, Op, Pred), first1, last1, first2, stencil, result, op, pred);                                                \
  }
THRUST_CDNA4_TRANSFORM_IF_NO_POLICY(THRUST_CDNA4_DEVICE_SYS, detail::enable_if_device)
THRUST_CDNA4_TRANSFORM_IF_NO_POLICY(THRUST_CDNA4_HOST_SYS, detail::enable_if_host)
#undef THRUST_CDNA4_TRANSFORM_IF_NO_POLICY
}  // namespace thrust
