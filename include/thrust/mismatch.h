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
template <class D, class It1, class It2, class Pred>
pair<It1, It2> mismatch(const system::cdna4::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, Pred pred) {
  const std::int64_t n = (std::int64_t)(last1 - first1);
  const std::int64_t at = system::cdna4::detail::reduce_index(
      exec.derived(), n,
      detail::differ_index<typename detail::unwrap_iterator<It1>::type, typename detail::unwrap_iterator<It2>::type, Pred>{
          detail::unwrap(first1), detail::unwrap(first2), pred, n},
      n, detail::min_index());
  return thrust::make_pair(first1 + at, first2 + at);
}
template <class It1, class It2, class Pred>
pair<It1, It2> mismatch(const system::cpp::detail::par_t&, It1 first1, It1 last1, It2 first2, Pred pred) {
  auto r = std::mismatch(first1, last1, first2, pred);
  return thrust::make_pair(r.first, r.second);
}
template <class Policy, class It1, class It2, detail::enable_if_policy<Policy> = 0>
pair<It1, It2> mismatch(const Policy& exec, It1 f1, It1 l1, It2 f2) { return mismatch(exec, f1, l1, f2, equal_to<>()); }
template <class It1, class It2, detail::enable_if_device<It1> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2) { return mismatch(device, f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2) { return mismatch(host, f1, l1, f2); }
template <class It1, class It2, class P, detail::enable_if_device<It1> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2, P p) { return mismatch(device, f1, l1, f2, p); }
template <class It1, class It2, class P, detail::enable_if_host<It1> = 0> pair<It1, It2> mismatch(It1 f1, It1 l1, It2 f2, P p) { return mismatch(host, f1, l1, f2, p); }
}  // namespace thrust
