// thrust::device_allocator (thrust/device_allocator.h): the default allocator of
// device_vector; storage comes from the library's caching pool.
#pragma once
#include <thrust/mr/allocator.h>
#include <thrust/system/cdna4/memory_resource.h>

namespace thrust {
template <class T>
class device_allocator : public mr::stateless_resource_allocator<T, system::cdna4::pool_memory_resource> {
 public:
  template <class U> struct rebind { typedef device_allocator<U> other; };
  device_allocator() = default;
  template <class U> device_allocator(const device_allocator<U>& o) : mr::stateless_resource_allocator<T, system::cdna4::pool_memory_resource>(o) {}
};
}  // namespace thrust
