// thrust::device_new (thrust/device_new.h): n objects of T in device memory — in storage the
// caller provides (placement form) or from thrust::device_malloc — each a copy of an exemplar
// (a value-initialised T when none is given).  Elements of device storage are trivially copyable,
// so construction is assignment (thrust/detail/device_new.inl does the same with
// uninitialized_fill).
#pragma once
#include <cstddef>
#include <thrust/device_malloc.h>
#include <thrust/device_ptr.h>
#include <thrust/uninitialized_fill.h>
namespace thrust {
template <class T>
device_ptr<T> device_new(device_ptr<void> p, const T& exemplar, const std::size_t n = 1) {
  device_ptr<T> result(static_cast<T*>(p.get()));
  thrust::uninitialized_fill(device, result, result + n, exemplar);
  return result;
}
template <class T>
device_ptr<T> device_new(device_ptr<void> p, const std::size_t n = 1) { return device_new<T>(p, T(), n); }
template <class T>
device_ptr<T> device_new(const std::size_t n = 1) {
  return device_new<T>(device_ptr<void>(static_cast<void*>(device_malloc<T>(n).get())), n);
}
}  // namespace thrust
