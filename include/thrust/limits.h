// <thrust/limits.h>: thrust::numeric_limits is the standard one.
#pragma once
#include <limits>
namespace thrust {
template <class T> using numeric_limits = std::numeric_limits<T>;
}  // namespace thrust
