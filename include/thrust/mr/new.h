// thrust::mr::new_delete_resource (thrust/mr/new.h): host memory from operator new.
#pragma once
#include <cstdlib>
#include <new>
#include <thrust/mr/memory_resource.h>

namespace thrust { namespace mr {
class new_delete_resource final : public memory_resource<> {
 public:
  void* do_allocate(std::size_t bytes, std::size_t alignment) override {
    if (alignment <= alignof(std::max_align_t)) return ::operator new(bytes);
    void* p = nullptr;
    if (posix_memalign(&p, alignment, bytes ? bytes : alignment) != 0) throw std::bad_alloc();
    return p;
  }
  void do_deallocate(void* p, std::size_t, std::size_t alignment) override {
    if (alignment <= alignof(std::max_align_t)) ::operator delete(p);
    else std::free(p);
  }
  bool do_is_equal(const memory_resource<>& other) const noexcept override { return dynamic_cast<const new_delete_resource*>(&other) != nullptr; }
};
}}  // namespace thrust::mr
