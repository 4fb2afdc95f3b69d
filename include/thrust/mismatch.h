// thrust::mismatch (thrust/mismatch.h): the first position at which two ranges differ.
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/pair.h>

namespace thrust {
namespace detail {
template <class A, class B, class Pred> struct differ_index {
  A a; B b; mutable Pred pred; std::int64_t n;
  THRUST_CDNA4_HD std::int64_t operator()(std::int64_t i) const { return pred(a[i], b[i]) ? n : i; }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/mismatch.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/mismatch.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It1, class It2, class Pred>
pair<It1, It2> mismatch(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, Pred pred) {
  return mismatch(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, pred);
}
template <class It1, class It2, class Pred>
pair<It1, It2> mismatch(const system::cpp::detail::par_t&, It1 first1, It1 last1, It2 first2, Pred pred) {
  auto r = std::mismatch(first1, last1, first2, pred);
  return thrust::make_pair(r.first, r.second);
}
namespace detail {
template <class Policy, class It1, class It2>
pair<It1, It2> composed_mismatch(const Policy& exec, It1 f1, It1 l1, It2 f2) { return mismatch(exec, f1, l1, f2, equal_to<>()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It1, class It2>
pair<It1, It2> mismatch(execution_policy<D_>& exec, It1 f1, It1 l1, It2 f2) { return thrust::detail::composed_mismatch(exec, f1, l1, f2); }
}}  // namespace system::cdna4
template <class D_, class It1, class It2>
pair<It1, It2> mismatch(const detail::execution_policy_base<D_>& exec, It1 f1, It1 l1, It2 f2) { return mismatch(detail::derived_cast(detail::strip_const(exec)), f1, l1, f2); }
template <class It1, class It2>
pair<It1, It2> mismatch(const system::cpp::detail::par_t& exec, It1 f1, It1 l1, It2 f2) { return detail::composed_mismatch(exec, f1, l1, f2); }
template <class It1, class It2, detail::enable_if_device<It1, It2> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2) { return mismatch(typename detail::implicit_policy<It1, It2>::type(), f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1, It2> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2) { return mismatch(host, f1, l1, f2); }
template <class It1, class It2, class P, detail::enable_if_device<It1, It2, P> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2, P p) { return mismatch(typename detail::implicit_policy<It1, It2, P>::type(), f1, l1, f2, p); }
template <class It1, class It2, class P, detail::enable_if_host<It1, It2, P> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2, P p) { return mismatch(host, f1, l1, f2, p); }
}  // namespace thrust
