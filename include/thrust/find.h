// thrust::find / find_if / find_if_not (thrust/find.h): the first position whose element
// satisfies the predicate, as a minimum over the matching indices.
#pragma once
#include <algorithm>
#include <thrust/count.h>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class It, class Pred, bool NEGATE> struct match_index {
  It p; mutable Pred pred; std::int64_t n;
  THRUST_CDNA4_HD std::int64_t operator()(std::int64_t i) const { return ((bool)pred(p[i]) != NEGATE) ? i : n; }
};
struct min_index {
  THRUST_CDNA4_HD std::int64_t operator()(std::int64_t a, std::int64_t b) const { return a < b ? a : b; }
};
template <bool NEGATE, class Policy, class It, class Pred>
It find_first(const Policy& exec, It first, It last, Pred pred) {
  const std::int64_t n = (std::int64_t)(last - first);
  typedef typename unwrap_iterator<It>::type U;
  const std::int64_t at = system::cdna4::detail::reduce_index(exec, n, match_index<U, Pred, NEGATE>{unwrap(first), pred, n}, n, min_index());
  return first + at;
}
template <class Pred> struct negated {
  mutable Pred pred;
  template <class T> THRUST_CDNA4_HD bool operator()(const T& x) const { return !pred(x); }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/find.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/find.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class Pred>
It find_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return find_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <class D, class It, class Pred>
It find_if_not(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return find_if_not(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <class It, class Pred> It find_if(const system::cpp::detail::par_t&, It first, It last, Pred pred) { return std::find_if(first, last, pred); }
template <class It, class Pred> It find_if_not(const system::cpp::detail::par_t&, It first, It last, Pred pred) { return std::find_if_not(first, last, pred); }
namespace detail {
template <class Policy, class It, class T>
It composed_find(const Policy& exec, It first, It last, const T& value) { return find_if(exec, first, last, detail::equals_value<T>{value}); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class T>
It find(execution_policy<D_>& exec, It first, It last, const T& value) { return thrust::detail::composed_find(exec, first, last, value); }
}}  // namespace system::cdna4
template <class D_, class It, class T>
It find(const detail::execution_policy_base<D_>& exec, It first, It last, const T& value) { return find(detail::derived_cast(detail::strip_const(exec)), first, last, value); }
template <class It, class T>
It find(const system::cpp::detail::par_t& exec, It first, It last, const T& value) { return detail::composed_find(exec, first, last, value); }

template <class It, class T, detail::enable_if_device<It, T> = 0> It find(It f, It l, const T& v) { return find(typename detail::implicit_policy<It, T>::type(), f, l, v); }
template <class It, class T, detail::enable_if_host<It, T> = 0> It find(It f, It l, const T& v) { return find(host, f, l, v); }
template <class It, class P, detail::enable_if_device<It, P> = 0> It find_if(It f, It l, P p) { return find_if(typename detail::implicit_policy<It, P>::type(), f, l, p); }
template <class It, class P, detail::enable_if_host<It, P> = 0> It find_if(It f, It l, P p) { return find_if(host, f, l, p); }
template <class It, class P, detail::enable_if_device<It, P> = 0> It find_if_not(It f, It l, P p) { return find_if_not(typename detail::implicit_policy<It, P>::type(), f, l, p); }
template <class It, class P, detail::enable_if_host<It, P> = 0> It find_if_not(It f, It l, P p) { return find_if_not(host, f, l, p); }
}  // namespace thrust
