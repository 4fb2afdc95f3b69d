// thrust::device_make_unique (thrust/device_make_unique.h): one T(args...) in device memory from
// thrust::device_allocator, owned by a std::unique_ptr that hands the storage back.
#pragma once
#include <utility>
#include <thrust/allocate_unique.h>
#include <thrust/device_allocator.h>
#include <thrust/device_new.h>
#include <thrust/device_ptr.h>
namespace thrust {
template <class T, class... Args>
auto device_make_unique(Args&&... args) -> decltype(uninitialized_allocate_unique<T>(device_allocator<T>{})) {
  auto p = uninitialized_allocate_unique<T>(device_allocator<T>{});
  device_new<T>(device_ptr<void>(static_cast<void*>(p.get().get())), T(std::forward<Args>(args)...));
  return p;
}
}  // namespace thrust
