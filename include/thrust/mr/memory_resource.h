// thrust::mr::memory_resource (thrust/mr/memory_resource.h:39-170): the polymorphic allocation
// interface; Pointer is void* for host resources and device_ptr<void> for device ones.
#pragma once
#include <cstddef>

namespace thrust { namespace mr {
template <class Pointer = void*>
class memory_resource {
 public:
  typedef Pointer pointer;
  virtual ~memory_resource() = default;
  pointer allocate(std::size_t bytes, std::size_t alignment = alignof(std::max_align_t)) { return do_allocate(bytes, alignment); }
  void deallocate(pointer p, std::size_t bytes, std::size_t alignment = alignof(std::max_align_t)) { do_deallocate(p, bytes, alignment); }
  bool is_equal(const memory_resource& other) const noexcept { return do_is_equal(other); }
  virtual pointer do_allocate(std::size_t bytes, std::size_t alignment) = 0;
  virtual void do_deallocate(pointer p, std::size_t bytes, std::size_t alignment) = 0;
  virtual bool do_is_equal(const memory_resource& other) const noexcept { return this == &other; }
};
template <class P>
bool operator==(const memory_resource<P>& a, const memory_resource<P>& b) noexcept { return &a == &b || a.is_equal(b); }
template <class P>
bool operator!=(const memory_resource<P>& a, const memory_resource<P>& b) noexcept { return !(a == b); }

// one resource object per type, created on first use (thrust/mr/memory_resource.h:196-212)
template <class MR>
MR* get_global_resource() {
  static MR resource;
  return &resource;
}
}}  // namespace thrust::mr
