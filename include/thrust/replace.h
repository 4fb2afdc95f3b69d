// thrust::replace / replace_if / replace_copy / replace_copy_if (thrust/replace.h).
#pragma once
#include <algorithm>
#include <thrust/count.h>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
// out[i] = pred(stencil[i]) ? value : in[i]
template <class In, class S, class Out, class Pred, class T> struct replace_body {
  In in; S stencil; Out out; Pred pred; T value;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    if (pred(stencil[i])) out[i] = value;
    else out[i] = in[i];
  }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/replace.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/replace.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class S, class Out, class Pred, class T>
Out replace_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, S stencil, Out result, Pred pred, const T& value) {
  return replace_copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, result, pred, value);
}
template <class In, class S, class Out, class Pred, class T>
Out replace_copy_if(const system::cpp::detail::par_t&, In first, In last, S stencil, Out result, Pred pred, const T& value) {
  for (; first != last; ++first, ++stencil, ++result) {
    if (pred(*stencil)) *result = value;
    else *result = *first;
  }
  return result;
}
namespace detail {
template <class Policy, class In, class Out, class Pred, class T>
Out composed_replace_copy_if(const Policy& exec, In first, In last, Out result, Pred pred, const T& value) {
  return replace_copy_if(exec, first, last, first, result, pred, value);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out, class Pred, class T>
Out replace_copy_if(execution_policy<D_>& exec, In first, In last, Out result, Pred pred, const T& value) { return thrust::detail::composed_replace_copy_if(exec, first, last, result, pred, value); }
}}  // namespace system::cdna4
template <class D_, class In, class Out, class Pred, class T>
Out replace_copy_if(const detail::execution_policy_base<D_>& exec, In first, In last, Out result, Pred pred, const T& value) { return replace_copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, result, pred, value); }
template <class In, class Out, class Pred, class T>
Out replace_copy_if(const system::cpp::detail::par_t& exec, In first, In last, Out result, Pred pred, const T& value) { return detail::composed_replace_copy_if(exec, first, last, result, pred, value); }
namespace detail {
template <class Policy, class In, class Out, class T>
Out composed_replace_copy(const Policy& exec, In first, In last, Out result, const T& old_value, const T& new_value) {
  return replace_copy_if(exec, first, last, first, result, detail::equals_value<T>{old_value}, new_value);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out, class T>
Out replace_copy(execution_policy<D_>& exec, In first, In last, Out result, const T& old_value, const T& new_value) { return thrust::detail::composed_replace_copy(exec, first, last, result, old_value, new_value); }
}}  // namespace system::cdna4
template <class D_, class In, class Out, class T>
Out replace_copy(const detail::execution_policy_base<D_>& exec, In first, In last, Out result, const T& old_value, const T& new_value) { return replace_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result, old_value, new_value); }
template <class In, class Out, class T>
Out replace_copy(const system::cpp::detail::par_t& exec, In first, In last, Out result, const T& old_value, const T& new_value) { return detail::composed_replace_copy(exec, first, last, result, old_value, new_value); }
namespace detail {
template <class Policy, class It, class Pred, class T>
void composed_replace_if(const Policy& exec, It first, It last, Pred pred, const T& value) { replace_copy_if(exec, first, last, first, first, pred, value); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred, class T>
void replace_if(execution_policy<D_>& exec, It first, It last, Pred pred, const T& value) { return thrust::detail::composed_replace_if(exec, first, last, pred, value); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred, class T>
void replace_if(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred, const T& value) { return replace_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred, value); }
template <class It, class Pred, class T>
void replace_if(const system::cpp::detail::par_t& exec, It first, It last, Pred pred, const T& value) { return detail::composed_replace_if(exec, first, last, pred, value); }
namespace detail {
template <class Policy, class It, class S, class Pred, class T>
void composed_replace_if(const Policy& exec, It first, It last, S stencil, Pred pred, const T& value) { replace_copy_if(exec, first, last, stencil, first, pred, value); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class S, class Pred, class T>
void replace_if(execution_policy<D_>& exec, It first, It last, S stencil, Pred pred, const T& value) { return thrust::detail::composed_replace_if(exec, first, last, stencil, pred, value); }
}}  // namespace system::cdna4
template <class D_, class It, class S, class Pred, class T>
void replace_if(const detail::execution_policy_base<D_>& exec, It first, It last, S stencil, Pred pred, const T& value) { return replace_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, pred, value); }
template <class It, class S, class Pred, class T>
void replace_if(const system::cpp::detail::par_t& exec, It first, It last, S stencil, Pred pred, const T& value) { return detail::composed_replace_if(exec, first, last, stencil, pred, value); }
namespace detail {
template <class Policy, class It, class T>
void composed_replace(const Policy& exec, It first, It last, const T& old_value, const T& new_value) {
  replace_copy_if(exec, first, last, first, first, detail::equals_value<T>{old_value}, new_value);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class T>
void replace(execution_policy<D_>& exec, It first, It last, const T& old_value, const T& new_value) { return thrust::detail::composed_replace(exec, first, last, old_value, new_value); }
}}  // namespace system::cdna4
template <class D_, class It, class T>
void replace(const detail::execution_policy_base<D_>& exec, It first, It last, const T& old_value, const T& new_value) { return replace(detail::derived_cast(detail::strip_const(exec)), first, last, old_value, new_value); }
template <class It, class T>
void replace(const system::cpp::detail::par_t& exec, It first, It last, const T& old_value, const T& new_value) { return detail::composed_replace(exec, first, last, old_value, new_value); }

#define THRUST_CDNA4_REPLACE(SYS, COND)                                                                                       \
  template <class It, class T, COND<It, T> = 0> void replace(It f, It l, const T& a, const T& b) { replace(SYS(It, T), f, l, a, b); }    \
  template <class It, class P, class T, COND<It, P, T> = 0> void replace_if(It f, It l, P p, const T& v) { replace_if(SYS(It, P, T), f, l, p, v); } \
  template <class It, class S, class P, class T, COND<It, S, P, T> = 0, class = typename std::iterator_traits<S>::iterator_category>    \
  void replace_if(It f, It l, S s, P p, const T& v) { replace_if(SYS(It, S, P, T), f, l, s, p, v); }                                        \
  template <class In, class Out, class T, COND<In, Out, T> = 0> Out replace_copy(In f, In l, Out o, const T& a, const T& b) { return replace_copy(SYS(In, Out, T), f, l, o, a, b); } \
  template <class In, class Out, class P, class T, COND<In, Out, P, T> = 0> Out replace_copy_if(In f, In l, Out o, P p, const T& v) { return replace_copy_if(SYS(In, Out, P, T), f, l, o, p, v); } \
  template <class In, class S, class Out, class P, class T, COND<In, S, Out, P, T> = 0> Out replace_copy_if(In f, In l, S s, Out o, P p, const T& v) { return replace_copy_if(SYS(In, S, Out, P, T), f, l, s, o, p, v); }
THRUST_CDNA4_REPLACE(THRUST_CDNA4_DEVICE_SYS, detail::enable_if_device)
THRUST_CDNA4_REPLACE(THRUST_CDNA4_HOST_SYS, detail::enable_if_host)
#undef THRUST_CDNA4_REPLACE
}  // namespace thrust
