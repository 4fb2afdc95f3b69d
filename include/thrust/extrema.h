// thrust::min_element / max_element / minmax_element (thrust/extrema.h) and thrust::min / max.
// A reduction over (value, position) pairs; among equal extrema the first position wins, for
// the minimum and for the maximum alike (thrust/system/detail/generic/extrema.inl).
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/detail/minmax.h>
#include <thrust/pair.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

#include <thrust/reduce.h>
#include <thrust/transform.h>
namespace thrust {

namespace detail {
// position -1: no element yet
template <class V> struct extremum {
  V lo; std::int64_t lo_at;
  V hi; std::int64_t hi_at;
};
template <class It, class V> struct extremum_at {
  It p;
  THRUST_CDNA4_HD extremum<V> operator()(std::int64_t i) const {
    const V v = p[i];
    return extremum<V>{v, i, v, i};
  }
};
template <class V, class Compare> struct extremum_merge {
  mutable Compare comp;
  THRUST_CDNA4_HD extremum<V> operator()(const extremum<V>& a, const extremum<V>& b) const {
    if (a.lo_at < 0) return b;
    if (b.lo_at < 0) return a;
    extremum<V> r = a;
    if (comp(b.lo, a.lo) || (!comp(a.lo, b.lo) && b.lo_at < a.lo_at)) { r.lo = b.lo; r.lo_at = b.lo_at; }
    if (comp(a.hi, b.hi) || (!comp(b.hi, a.hi) && b.hi_at < a.hi_at)) { r.hi = b.hi; r.hi_at = b.hi_at; }
    return r;
  }
};
template <class Policy, class It, class Compare>
extremum<typename value_of<It>::type> extrema_of(const Policy& exec, It first, It last, Compare comp) {
  typedef typename value_of<It>::type V;
  typedef typename unwrap_iterator<It>::type U;
  return system::cdna4::detail::reduce_index(exec, (std::int64_t)(last - first), extremum_at<U, V>{unwrap(first)},
                                             extremum<V>{V(), -1, V(), -1}, extremum_merge<V, Compare>{comp});
}
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/extrema.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/extrema.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class Compare>
It min_element(const detail::execution_policy_base<D>& exec, It first, It last, Compare comp) {
  return min_element(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <class D, class It, class Compare>
It max_element(const detail::execution_policy_base<D>& exec, It first, It last, Compare comp) {
  return max_element(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <class D, class It, class Compare>
pair<It, It> minmax_element(const detail::execution_policy_base<D>& exec, It first, It last, Compare comp) {
  return minmax_element(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <class It, class Compare> It min_element(const system::cpp::detail::par_t&, It first, It last, Compare comp) { return std::min_element(first, last, comp); }
template <class It, class Compare> It max_element(const system::cpp::detail::par_t&, It first, It last, Compare comp) { return std::max_element(first, last, comp); }
template <class It, class Compare>
pair<It, It> minmax_element(const system::cpp::detail::par_t&, It first, It last, Compare comp) {
  return thrust::make_pair(std::min_element(first, last, comp), std::max_element(first, last, comp));  // the FIRST maximum
}
#define THRUST_CDNA4_EXTREMA(NAME, RET)                                                                                     \
  template <class D, class It> RET NAME(const detail::execution_policy_base<D>& exec, It f, It l) { return NAME(detail::derived_cast(detail::strip_const(exec)), f, l); } \
  template <class It> RET NAME(const system::cpp::detail::par_t& exec, It f, It l) { return NAME(exec, f, l, less<>()); }     \
  template <class It, detail::enable_if_device<It> = 0> RET NAME(It f, It l) { return NAME(typename detail::implicit_policy<It>::type(), f, l); }                    \
  template <class It, detail::enable_if_host<It> = 0> RET NAME(It f, It l) { return NAME(host, f, l); }                        \
  template <class It, class C, detail::enable_if_device<It, C> = 0> RET NAME(It f, It l, C c) { return NAME(typename detail::implicit_policy<It, C>::type(), f, l, c); }  \
  template <class It, class C, detail::enable_if_host<It, C> = 0> RET NAME(It f, It l, C c) { return NAME(host, f, l, c); }
THRUST_CDNA4_EXTREMA(min_element, It)
THRUST_CDNA4_EXTREMA(max_element, It)
#define THRUST_CDNA4_PAIR_OF_IT pair<It, It>
THRUST_CDNA4_EXTREMA(minmax_element, THRUST_CDNA4_PAIR_OF_IT)
#undef THRUST_CDNA4_PAIR_OF_IT
#undef THRUST_CDNA4_EXTREMA
}  // namespace thrust
