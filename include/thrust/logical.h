// thrust::all_of / any_of / none_of (thrust/logical.h), on find_if as in the reference
// (thrust/system/detail/generic/logical.h).
#pragma once
#include <thrust/find.h>

namespace thrust {
namespace detail {
template <class Policy, class It, class Pred>
bool composed_all_of(const Policy& exec, It first, It last, Pred pred) { return find_if_not(exec, first, last, pred) == last; }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred>
bool all_of(execution_policy<D_>& exec, It first, It last, Pred pred) { return thrust::detail::composed_all_of(exec, first, last, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred>
bool all_of(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred) { return all_of(detail::derived_cast(detail::strip_const(exec)), first, last, pred); }
template <class It, class Pred>
bool all_of(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_all_of(exec, first, last, pred); }
namespace detail {
template <class Policy, class It, class Pred>
bool composed_any_of(const Policy& exec, It first, It last, Pred pred) { return find_if(exec, first, last, pred) != last; }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred>
bool any_of(execution_policy<D_>& exec, It first, It last, Pred pred) { return thrust::detail::composed_any_of(exec, first, last, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred>
bool any_of(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred) { return any_of(detail::derived_cast(detail::strip_const(exec)), first, last, pred); }
template <class It, class Pred>
bool any_of(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_any_of(exec, first, last, pred); }
namespace detail {
template <class Policy, class It, class Pred>
bool composed_none_of(const Policy& exec, It first, It last, Pred pred) { return !any_of(exec, first, last, pred); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred>
bool none_of(execution_policy<D_>& exec, It first, It last, Pred pred) { return thrust::detail::composed_none_of(exec, first, last, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred>
bool none_of(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred) { return none_of(detail::derived_cast(detail::strip_const(exec)), first, last, pred); }
template <class It, class Pred>
bool none_of(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_none_of(exec, first, last, pred); }
#define THRUST_CDNA4_LOGICAL(NAME)                                                                                   \
  template <class It, class P, detail::enable_if_device<It, P> = 0> bool NAME(It f, It l, P p) { return NAME(typename detail::implicit_policy<It, P>::type(), f, l, p); } \
  template <class It, class P, detail::enable_if_host<It, P> = 0> bool NAME(It f, It l, P p) { return NAME(host, f, l, p); }
THRUST_CDNA4_LOGICAL(all_of)
THRUST_CDNA4_LOGICAL(any_of)
THRUST_CDNA4_LOGICAL(none_of)
#undef THRUST_CDNA4_LOGICAL
}  // namespace thrust
