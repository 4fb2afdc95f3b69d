// The cdna4 device system's malloc and free (the counterpart of
// thrust/system/cuda/detail/malloc_and_free.h:53-116, which calls cudaMalloc / cudaFree on every
// call): blocks come from the library's cached pool and are ordered on the policy's stream.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/system/cdna4/detail/core.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class D>
device_ptr<void> malloc(const execution_policy<D>& exec, std::size_t n) {
  return device_ptr<void>(detail::malloc_bytes(n, detail::stream_of(exec.derived())));  // throws bad_alloc
}
template <class T, class D>
device_ptr<T> malloc(const execution_policy<D>& exec, std::size_t n) {
  return device_ptr<T>(static_cast<T*>(detail::malloc_bytes(n * sizeof(T), detail::stream_of(exec.derived()))));
}
template <class D, class Pointer>
void free(const execution_policy<D>& exec, Pointer ptr) {
  detail::free_bytes(const_cast<void*>(static_cast<const void*>(thrust::raw_pointer_cast(ptr))), detail::stream_of(exec.derived()));
}
}}  // namespace system::cdna4
}  // namespace thrust
