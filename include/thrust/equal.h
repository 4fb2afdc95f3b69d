// thrust::equal (thrust/equal.h): no position at which the two ranges differ.
#pragma once
#include <thrust/mismatch.h>

namespace thrust {
namespace detail {
template <class Policy, class It1, class It2, class Pred>
bool composed_equal(const Policy& exec, It1 first1, It1 last1, It2 first2, Pred pred) { return mismatch(exec, first1, last1, first2, pred).first == last1; }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It1, class It2, class Pred>
bool equal(execution_policy<D_>& exec, It1 first1, It1 last1, It2 first2, Pred pred) { return thrust::detail::composed_equal(exec, first1, last1, first2, pred); }
}}  // namespace system::cdna4
template <class D_, class It1, class It2, class Pred>
bool equal(const detail::execution_policy_base<D_>& exec, It1 first1, It1 last1, It2 first2, Pred pred) { return equal(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, pred); }
template <class It1, class It2, class Pred>
bool equal(const system::cpp::detail::par_t& exec, It1 first1, It1 last1, It2 first2, Pred pred) { return detail::composed_equal(exec, first1, last1, first2, pred); }
namespace detail {
template <class Policy, class It1, class It2>
bool composed_equal(const Policy& exec, It1 first1, It1 last1, It2 first2) { return equal(exec, first1, last1, first2, equal_to<>()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It1, class It2>
bool equal(execution_policy<D_>& exec, It1 first1, It1 last1, It2 first2) { return thrust::detail::composed_equal(exec, first1, last1, first2); }
}}  // namespace system::cdna4
template <class D_, class It1, class It2>
bool equal(const detail::execution_policy_base<D_>& exec, It1 first1, It1 last1, It2 first2) { return equal(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2); }
template <class It1, class It2>
bool equal(const system::cpp::detail::par_t& exec, It1 first1, It1 last1, It2 first2) { return detail::composed_equal(exec, first1, last1, first2); }
template <class It1, class It2, detail::enable_if_device<It1, It2> = 0> bool equal(It1 f1, It1 l1, It2 f2) { return equal(typename detail::implicit_policy<It1, It2>::type(), f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1, It2> = 0> bool equal(It1 f1, It1 l1, It2 f2) { return equal(host, f1, l1, f2); }
template <class It1, class It2, class P, detail::enable_if_device<It1, It2, P> = 0> bool equal(It1 f1, It1 l1, It2 f2, P p) { return equal(typename detail::implicit_policy<It1, It2, P>::type(), f1, l1, f2, p); }
template <class It1, class It2, class P, detail::enable_if_host<It1, It2, P> = 0> bool equal(It1 f1, It1 l1, It2 f2, P p) { return equal(host, f1, l1, f2, p); }
}  // namespace thrust
