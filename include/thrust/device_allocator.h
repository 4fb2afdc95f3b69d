// thrust::device_allocator (thrust/device_allocator.h): the default allocator of
// device_vector; storage comes from the library's caching pool.
#pragma once
#include <thrust/mr/allocator.h>
#include <thrust/system/cdna4/memory_resource.h>

namespace thrust {
// A device resource seen as a resource of device_ptr<void> (thrust/device_allocator.h:44-83).  The
// resources of this system already hand out device_ptr<void>, so this forwards.
template <class Upstream>
class device_ptr_memory_resource final : public mr::memory_resource<device_ptr<void>> {
 public:
  device_ptr_memory_resource() : upstream_(mr::get_global_resource<Upstream>()) {}
  explicit device_ptr_memory_resource(Upstream* upstream) : upstream_(upstream) {}
  device_ptr<void> do_allocate(std::size_t bytes, std::size_t alignment) override { return device_ptr<void>(upstream_->allocate(bytes, alignment)); }
  void do_deallocate(device_ptr<void> p, std::size_t bytes, std::size_t alignment) override { upstream_->deallocate(p, bytes, alignment); }
  bool do_is_equal(const mr::memory_resource<device_ptr<void>>& other) const noexcept override {
    const device_ptr_memory_resource* o = dynamic_cast<const device_ptr_memory_resource*>(&other);
    return o && *upstream_ == *o->upstream_;
  }
 private:
  Upstream* upstream_;
};
template <class T>
class device_allocator : public mr::stateless_resource_allocator<T, system::cdna4::pool_memory_resource> {
 public:
  template <class U> struct rebind { typedef device_allocator<U> other; };
  device_allocator() = default;
  template <class U> device_allocator(const device_allocator<U>& o) : mr::stateless_resource_allocator<T, system::cdna4::pool_memory_resource>(o) {}
};
}  // namespace thrust
