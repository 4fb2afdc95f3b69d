// <thrust/limits.h>: thrust::numeric_limits — the standard limits under a class template of
// thrust's own, which user code may specialise for its number-like types (thrust/limits.h:14-19).
#pragma once
#include <limits>
namespace thrust {
template <class T> struct numeric_limits : std::numeric_limits<T> {};
}  // namespace thrust
