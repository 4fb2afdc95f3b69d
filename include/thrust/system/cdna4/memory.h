// thrust::cdna4::malloc / free / allocator / universal_allocator (the counterpart of
// thrust/system/cuda/memory.h:41-112): device memory of the cdna4 system, from the library's cached,
// stream-ordered pool.
#pragma once
#include <thrust/device_allocator.h>
#include <thrust/system/cdna4/detail/malloc_and_free.h>
#include <thrust/system/cdna4/memory_resource.h>
#include <thrust/system/cdna4/pointer.h>
#include <thrust/universal_allocator.h>
namespace thrust {
namespace system { namespace cdna4 {
inline pointer<void> malloc(std::size_t n) { return malloc(par, n); }
template <class T> inline pointer<T> malloc(std::size_t n) { return pointer<T>(static_cast<T*>(malloc(par, n * sizeof(T)).get())); }
inline void free(pointer<void> p) { free(par, p); }
template <class T> using allocator = thrust::device_allocator<T>;
template <class T> using universal_allocator = thrust::universal_allocator<T>;
}}  // namespace system::cdna4
namespace cdna4 {
using thrust::system::cdna4::allocator;
using thrust::system::cdna4::free;
using thrust::system::cdna4::malloc;
using thrust::system::cdna4::universal_allocator;
}  // namespace cdna4
}  // namespace thrust
