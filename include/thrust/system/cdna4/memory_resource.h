// Memory resources of the cdna4 system (thrust/system/cuda/memory_resource.h:46-120,
// thrust/mr/device_memory_resource.h): device memory straight from the driver, and the
// library's stream-ordered caching pool — the one every algorithm's temporary storage and
// device_vector use — as a resource that user containers and pools can share.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/mr/memory_resource.h>
#include <thrust/system/cdna4/detail/core.h>

namespace thrust { namespace system { namespace cdna4 {
// hipMalloc / hipFree on every call
class memory_resource final : public thrust::mr::memory_resource<thrust::device_ptr<void>> {
 public:
  thrust::device_ptr<void> do_allocate(std::size_t bytes, std::size_t) override {
    void* p = nullptr;
    const int rc = thrust_cdna4_malloc_direct(&p, bytes);
    if (rc != 0) throw thrust::system::detail::bad_alloc(thrust_cdna4_error_string(rc));
    return thrust::device_ptr<void>(p);
  }
  void do_deallocate(thrust::device_ptr<void> p, std::size_t, std::size_t) override {
    detail::throw_on_error(thrust_cdna4_free_direct(p.get()), "cdna4::memory_resource: free");
  }
  bool do_is_equal(const thrust::mr::memory_resource<thrust::device_ptr<void>>& other) const noexcept override {
    return dynamic_cast<const memory_resource*>(&other) != nullptr;
  }
};
// The library's pool: blocks are cached in power-of-two size classes and reuse is ordered on the
// stream given here (a block freed on one stream is reused on another only after the free has
// been reached there).
class pool_memory_resource final : public thrust::mr::memory_resource<thrust::device_ptr<void>> {
 public:
  explicit pool_memory_resource(void* stream = nullptr) : stream_(stream) {}
  thrust::device_ptr<void> do_allocate(std::size_t bytes, std::size_t) override {
    return thrust::device_ptr<void>(detail::malloc_bytes(bytes, stream_));
  }
  void do_deallocate(thrust::device_ptr<void> p, std::size_t, std::size_t) override { detail::free_bytes(p.get(), stream_); }
  bool do_is_equal(const thrust::mr::memory_resource<thrust::device_ptr<void>>& other) const noexcept override {
    const pool_memory_resource* o = dynamic_cast<const pool_memory_resource*>(&other);
    return o && o->stream_ == stream_;
  }
  // cached + handed-out bytes of the pool on the current device, and a way to give the cache back
  static std::size_t bytes_held() { return thrust_cdna4_pool_bytes(); }
  static void trim() { detail::throw_on_error(thrust_cdna4_pool_trim(), "cdna4::pool_memory_resource: trim"); }
 private:
  void* stream_;
};
// Memory that host code and device code can both address
// (thrust/system/cuda/memory_resource.h:118-125): managed memory, or page-locked host memory that
// the device reaches over the bus.  Pointers are device_ptr, like every pointer of this system;
// raw_pointer_cast of one may also be dereferenced on the host.
template <bool HOST_PINNED>
class universal_resource final : public thrust::mr::memory_resource<thrust::device_ptr<void>> {
 public:
  thrust::device_ptr<void> do_allocate(std::size_t bytes, std::size_t) override {
    void* p = nullptr;
    const int rc = thrust_cdna4_malloc_universal(&p, bytes, HOST_PINNED ? 1 : 0);
    if (rc != 0) throw thrust::system::detail::bad_alloc(thrust_cdna4_error_string(rc));
    return thrust::device_ptr<void>(p);
  }
  void do_deallocate(thrust::device_ptr<void> p, std::size_t, std::size_t) override {
    detail::throw_on_error(thrust_cdna4_free_universal(p.get(), HOST_PINNED ? 1 : 0), "cdna4::universal_memory_resource: free");
  }
  bool do_is_equal(const thrust::mr::memory_resource<thrust::device_ptr<void>>& other) const noexcept override {
    return dynamic_cast<const universal_resource*>(&other) != nullptr;
  }
};
typedef universal_resource<false> universal_memory_resource;
typedef universal_resource<true> universal_host_pinned_memory_resource;
}}  // namespace system::cdna4
typedef system::cdna4::memory_resource device_memory_resource;
typedef system::cdna4::universal_memory_resource universal_memory_resource;
typedef system::cdna4::universal_host_pinned_memory_resource universal_host_pinned_memory_resource;
}  // namespace thrust
