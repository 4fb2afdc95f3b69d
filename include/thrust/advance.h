// thrust::advance / next / prev (thrust/advance.h).
#pragma once
#include <iterator>
namespace thrust {
template <class It, class Distance> inline void advance(It& i, Distance n) { std::advance(i, n); }
template <class It> inline It next(It i, typename std::iterator_traits<It>::difference_type n = 1) { std::advance(i, n); return i; }
template <class It> inline It prev(It i, typename std::iterator_traits<It>::difference_type n = 1) { std::advance(i, -n); return i; }
}  // namespace thrust
