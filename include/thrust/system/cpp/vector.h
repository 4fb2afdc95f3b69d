// thrust::cpp::vector (thrust/system/cpp/vector.h): the host system's vector is thrust::host_vector.
#pragma once
#include <thrust/host_vector.h>
#include <thrust/system/cpp/memory.h>
namespace thrust {
namespace system { namespace cpp {
template <class T, class Allocator = std::allocator<T>> using vector = thrust::host_vector<T, Allocator>;
template <class T, class Allocator = std::allocator<T>> using universal_vector = thrust::host_vector<T, Allocator>;
}}  // namespace system::cpp
namespace cpp {
using thrust::system::cpp::universal_vector;
using thrust::system::cpp::vector;
}  // namespace cpp
}  // namespace thrust
