// thrust::pair (thrust/pair.h).
#pragma once
#include <utility>
namespace thrust {
template <class A, class B>
using pair = std::pair<A, B>;
using std::make_pair;
}  // namespace thrust
