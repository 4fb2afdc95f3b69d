// thrust::mr::fancy_pointer_resource (thrust/mr/fancy_pointer_resource.h): an upstream resource
// seen through another pointer type (e.g. a resource of raw void* as one of device_ptr<void>).
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/mr/memory_resource.h>
namespace thrust { namespace mr {
namespace detail {
inline void* raw_of(void* p) { return p; }
template <class T> inline void* raw_of(thrust::device_ptr<T> p) { return (void*)p.get(); }
template <class Pointer> struct pointer_from_raw { static Pointer make(void* p) { return Pointer(p); } };
template <> struct pointer_from_raw<void*> { static void* make(void* p) { return p; } };
}  // namespace detail
template <class Upstream, class Pointer>
class fancy_pointer_resource final : public memory_resource<Pointer> {
 public:
  fancy_pointer_resource() : upstream_(get_global_resource<Upstream>()) {}
  explicit fancy_pointer_resource(Upstream* upstream) : upstream_(upstream) {}
  Pointer do_allocate(std::size_t bytes, std::size_t alignment) override {
    return detail::pointer_from_raw<Pointer>::make(detail::raw_of(upstream_->allocate(bytes, alignment)));
  }
  void do_deallocate(Pointer p, std::size_t bytes, std::size_t alignment) override {
    upstream_->deallocate(detail::pointer_from_raw<typename Upstream::pointer>::make(detail::raw_of(p)), bytes, alignment);
  }
  bool do_is_equal(const memory_resource<Pointer>& other) const noexcept override {
    const fancy_pointer_resource* o = dynamic_cast<const fancy_pointer_resource*>(&other);
    return o && *upstream_ == *o->upstream_;
  }
 private:
  Upstream* upstream_;
};
}}  // namespace thrust::mr
