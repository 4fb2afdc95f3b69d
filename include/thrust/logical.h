// thrust::all_of / any_of / none_of (thrust/logical.h), on find_if as in the reference
// (thrust/system/detail/generic/logical.h).
#pragma once
#include <thrust/find.h>

namespace thrust {
template <class Policy, class It, class Pred, detail::enable_if_policy<Policy> = 0>
bool all_of(const Policy& exec, It first, It last, Pred pred) { return find_if_not(exec, first, last, pred) == last; }
template <class Policy, class It, class Pred, detail::enable_if_policy<Policy> = 0>
bool any_of(const Policy& exec, It first, It last, Pred pred) { return find_if(exec, first, last, pred) != last; }
template <class Policy, class It, class Pred, detail::enable_if_policy<Policy> = 0>
bool none_of(const Policy& exec, It first, It last, Pred pred) { return !any_of(exec, first, last, pred); }
#define THRUST_CDNA4_LOGICAL(NAME)                                                                                   \
  template <class It, class P, detail::enable_if_device<It, P> = 0> bool NAME(It f, It l, P p) { return NAME(device, f, l, p); } \
  template <class It, class P, detail::enable_if_host<It, P> = 0> bool NAME(It f, It l, P p) { return NAME(host, f, l, p); }
THRUST_CDNA4_LOGICAL(all_of)
THRUST_CDNA4_LOGICAL(any_of)
THRUST_CDNA4_LOGICAL(none_of)
#undef THRUST_CDNA4_LOGICAL
}  // namespace thrust
