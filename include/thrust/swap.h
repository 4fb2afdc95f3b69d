// thrust::swap and thrust::swap_ranges (thrust/swap.h).
#pragma once
#include <algorithm>
#include <utility>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
template <class A, class B> THRUST_CDNA4_HD inline void swap(A& a, B& b) {
  A t = a;
  a = b;
  b = t;
}
namespace detail {
template <class A, class B> struct swap_body {
  A a; B b;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    typename std::iterator_traits<A>::value_type t = a[i];
    a[i] = b[i];
    b[i] = t;
  }
};
}  // namespace detail
template <class D, class It1, class It2>
It2 swap_ranges(const system::cdna4::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2) {
  const std::int64_t n = (std::int64_t)(last1 - first1);
  system::cdna4::detail::for_each_index(
      exec.derived(), n,
      detail::swap_body<typename detail::unwrap_iterator<It1>::type, typename detail::unwrap_iterator<It2>::type>{detail::unwrap(first1), detail::unwrap(first2)},
      "swap_ranges: failed to synchronize");
  return first2 + n;
}
template <class It1, class It2> It2 swap_ranges(const system::cpp::detail::par_t&, It1 f1, It1 l1, It2 f2) { return std::swap_ranges(f1, l1, f2); }
template <class It1, class It2, detail::enable_if_device<It1> = 0> It2 swap_ranges(It1 f1, It1 l1, It2 f2) { return swap_ranges(device, f1, l1, f2); }
template <class It1, class It2, detail::enable_if_host<It1> = 0> It2 swap_ranges(It1 f1, It1 l1, It2 f2) { return swap_ranges(host, f1, l1, f2); }
}  // namespace thrust
