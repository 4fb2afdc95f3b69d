// Swapping two objects of one type the way generic code must (thrust/detail/swap.h, thrust/swap.h:
// "swap(a, b)" by an unqualified call): a swap that the type's author provides in the type's
// namespace is found through the arguments and preferred; assignment through a temporary otherwise.
// Host and device code both use it: std::swap is a host function.
#pragma once
#include <thrust/detail/hd.h>

namespace thrust {
namespace detail {
namespace swap_fallback {
template <class T>
THRUST_CDNA4_HD inline void swap(T& a, T& b) {
  T t = a;
  a = b;
  b = t;
}
}  // namespace swap_fallback
template <class T>
THRUST_CDNA4_HD inline void adl_swap(T& a, T& b) {
  using swap_fallback::swap;
  swap(a, b);
}
}  // namespace detail
}  // namespace thrust
