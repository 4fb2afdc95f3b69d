// thrust::equal (thrust/equal.h): no position at which the two ranges differ.
#pragma once
#include <thrust/mismatch.h>

namespace thrust {
template <class Policy, class It1, class It2, class Pred, detail::enable_if_policy<Policy> = 0>
bool equal(const Policy& exec, It1 first1, It1 last1, It2 first2, Pred pred) { return mismatch(exec, first1, last1, first2, pred).first == last1; }
template <class Policy, class It1, class It2, detail::enable_if_policy<Policy> = 0>
bool equal(const Policy& exec, It1 first1, It1 last1, It2 first2) { return equal(exec, first1, last1, first2, equal_to<>()); }
template <class It1, class It2, detail::enable_if_device<It1, It2> = 0> bool equal(It1 f1, It1 l1, It2 f2) { return equal(device, f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1, It2> = 0> bool equal(It1 f1, It1 l1, It2 f2) { return equal(host, f1, l1, f2); }
template <class It1, class It2, class P, detail::enable_if_device<It1, It2, P> = 0> bool equal(It1 f1, It1 l1, It2 f2, P p) { return equal(device, f1, l1, f2, p); }
template <class It1, class It2, class P, detail::enable_if_host<It1, It2, P> = 0> bool equal(It1 f1, It1 l1, It2 f2, P p) { return equal(host, f1, l1, f2, p); }
}  // namespace thrust
