// thrust::mr::polymorphic_adaptor_resource (thrust/mr/polymorphic_adaptor.h): a resource of a
// fixed type that forwards to any resource with the same pointer type through the virtual
// interface, so one allocator type (polymorphic_allocator in <thrust/mr/allocator.h>) can draw
// from resources chosen at run time.
#pragma once
#include <thrust/mr/memory_resource.h>
namespace thrust { namespace mr {
template <class Pointer = void*>
class polymorphic_adaptor_resource final : public memory_resource<Pointer> {
 public:
  polymorphic_adaptor_resource(memory_resource<Pointer>* upstream) : upstream_(upstream) {}
  Pointer do_allocate(std::size_t bytes, std::size_t alignment) override { return upstream_->allocate(bytes, alignment); }
  void do_deallocate(Pointer p, std::size_t bytes, std::size_t alignment) override { upstream_->deallocate(p, bytes, alignment); }
  bool do_is_equal(const memory_resource<Pointer>& other) const noexcept override {
    const polymorphic_adaptor_resource* o = dynamic_cast<const polymorphic_adaptor_resource*>(&other);
    return upstream_->is_equal(o ? *o->upstream_ : other);
  }
  memory_resource<Pointer>* upstream_resource() const { return upstream_; }
 private:
  memory_resource<Pointer>* upstream_;
};
}}  // namespace thrust::mr
