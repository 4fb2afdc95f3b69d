// thrust::get_per_device_resource / per_device_allocator (thrust/per_device_resource.h): one
// instance of a memory resource type per device, for the device that is current when it is asked
// for (thrust/system/cuda/detail/per_device_resource.h keeps one per CUDA device the same way).
#pragma once
#include <map>
#include <memory>
#include <mutex>
#include <thrust/execution_policy.h>
#include <thrust/mr/allocator.h>
namespace thrust {
namespace detail {
template <class MR>
MR* per_device_resource_of(int device) {
  static std::mutex mutex;
  static std::map<int, std::unique_ptr<MR>> resources;
  std::lock_guard<std::mutex> lock(mutex);
  std::unique_ptr<MR>& slot = resources[device];
  if (!slot) slot.reset(new MR());
  return slot.get();
}
}  // namespace detail
template <class MR, class DerivedPolicy>
MR* get_per_device_resource(const detail::execution_policy_base<DerivedPolicy>&) {
  int device = 0;
  system::cdna4::detail::throw_on_error(thrust_cdna4_get_device(&device), "get_per_device_resource");
  return detail::per_device_resource_of<MR>(device);
}
template <class MR>
MR* get_per_device_resource(const system::cpp::detail::par_t&) { return mr::get_global_resource<MR>(); }

template <class T, class Upstream, class ExecutionPolicy>
class per_device_allocator : public mr::allocator<T, Upstream> {
  typedef mr::allocator<T, Upstream> base;
 public:
  template <class U> struct rebind { typedef per_device_allocator<U, Upstream, ExecutionPolicy> other; };
  per_device_allocator() : base(get_per_device_resource<Upstream>(ExecutionPolicy())) {}
  per_device_allocator(const per_device_allocator& other) : base(other) {}
  template <class U> per_device_allocator(const per_device_allocator<U, Upstream, ExecutionPolicy>& other) : base(other) {}
};
}  // namespace thrust
