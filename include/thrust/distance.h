// thrust::distance (thrust/distance.h).
#pragma once
#include <iterator>
namespace thrust {
template <class It>
inline typename std::iterator_traits<It>::difference_type distance(It first, It last) { return std::distance(first, last); }
}  // namespace thrust
