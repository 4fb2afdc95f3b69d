// thrust::universal_allocator / universal_ptr (thrust/universal_allocator.h): storage that host
// and device code can both address, from the system's managed-memory resource.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/mr/allocator.h>
#include <thrust/system/cdna4/memory_resource.h>
namespace thrust {
template <class T>
class universal_allocator : public mr::stateless_resource_allocator<T, system::cdna4::universal_memory_resource> {
  typedef mr::stateless_resource_allocator<T, system::cdna4::universal_memory_resource> base;
 public:
  template <class U> struct rebind { typedef universal_allocator<U> other; };
  universal_allocator() = default;
  template <class U> universal_allocator(const universal_allocator<U>& o) : base(o) {}
};
// a pointer into universal memory: a device_ptr (the algorithms take it as a device range) whose
// raw pointer the host may dereference as well
template <class T> using universal_ptr = device_ptr<T>;
}  // namespace thrust
