// thrust::min / thrust::max of two values (thrust/detail/minmax.h; the reference's vector headers
// bring them along, and existing code calls them without naming a header).
#pragma once
#include <thrust/detail/hd.h>
namespace thrust {
template <class T> THRUST_CDNA4_HD constexpr const T& min(const T& a, const T& b) { return b < a ? b : a; }
template <class T> THRUST_CDNA4_HD constexpr const T& max(const T& a, const T& b) { return a < b ? b : a; }
template <class T, class Compare> THRUST_CDNA4_HD constexpr const T& min(const T& a, const T& b, Compare comp) { return comp(b, a) ? b : a; }
template <class T, class Compare> THRUST_CDNA4_HD constexpr const T& max(const T& a, const T& b, Compare comp) { return comp(a, b) ? b : a; }
}  // namespace thrust
