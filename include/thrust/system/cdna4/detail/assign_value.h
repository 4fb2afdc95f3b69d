// The cdna4 device system's assign_value (the counterpart of
// thrust/system/cuda/detail/assign_value.h): one element copied to device memory, from device or
// from host memory, complete when the call returns.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/system/cdna4/detail/core.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class D, class T, class U>
void assign_value(const execution_policy<D>& exec, device_ptr<T> dst, device_ptr<U> src) {
  static_assert(std::is_same<typename std::remove_const<U>::type, T>::value, "assign_value: one element type");
  void* s = detail::stream_of(exec.derived());
  detail::throw_on_error(thrust_cdna4_memcpy_dtod(dst.get(), src.get(), sizeof(T), s), "assign_value");
  detail::throw_on_error(thrust_cdna4_stream_synchronize(s), "assign_value");
}
template <class D, class T, class U>
void assign_value(const execution_policy<D>& exec, device_ptr<T> dst, U* src) {  // from host memory
  static_assert(std::is_same<typename std::remove_const<U>::type, T>::value, "assign_value: one element type");
  void* s = detail::stream_of(exec.derived());
  detail::throw_on_error(thrust_cdna4_memcpy_htod(dst.get(), src, sizeof(T), s), "assign_value");
  detail::throw_on_error(thrust_cdna4_stream_synchronize(s), "assign_value");
}
}}  // namespace system::cdna4
}  // namespace thrust
