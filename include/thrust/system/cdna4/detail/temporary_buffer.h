// The cdna4 device system's temporary buffers (the reference's device system leaves this file empty
// and inherits thrust/system/detail/generic/temporary_buffer.inl:34-79, which calls the system's
// malloc): a buffer of n elements from the cached pool, ordered on the policy's stream.  The
// algorithms' own temporaries go through temporary_storage (core.h), which also serves
// thrust::device(allocator).
#pragma once
#include <cstddef>
#include <thrust/pair.h>
#include <thrust/system/cdna4/detail/malloc_and_free.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class T, class D>
thrust::pair<device_ptr<T>, std::ptrdiff_t> get_temporary_buffer(const execution_policy<D>& exec, std::ptrdiff_t n) {
  if (n <= 0) return thrust::pair<device_ptr<T>, std::ptrdiff_t>(device_ptr<T>(), 0);
  return thrust::pair<device_ptr<T>, std::ptrdiff_t>(malloc<T>(exec, (std::size_t)n), n);
}
template <class D, class Pointer>
void return_temporary_buffer(const execution_policy<D>& exec, Pointer p, std::ptrdiff_t) { free(exec, p); }
}}  // namespace system::cdna4
}  // namespace thrust
