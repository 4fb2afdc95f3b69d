// thrust::cpp::malloc / free / allocator (thrust/system/cpp/memory.h): host memory of the host system.
#pragma once
#include <cstdlib>
#include <memory>
#include <thrust/system/cpp/memory_resource.h>
#include <thrust/system/cpp/pointer.h>
namespace thrust {
namespace system { namespace cpp {
inline void* malloc(std::size_t n) { return std::malloc(n); }
template <class T> inline T* malloc(std::size_t n) { return static_cast<T*>(std::malloc(n * sizeof(T))); }
inline void free(void* p) { std::free(p); }
template <class T> using allocator = std::allocator<T>;
template <class T> using universal_allocator = std::allocator<T>;
}}  // namespace system::cpp
namespace cpp {
using thrust::system::cpp::allocator;
using thrust::system::cpp::free;
using thrust::system::cpp::malloc;
using thrust::system::cpp::universal_allocator;
}  // namespace cpp
}  // namespace thrust
