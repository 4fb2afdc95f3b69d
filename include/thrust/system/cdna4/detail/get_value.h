// The cdna4 device system's get_value (the counterpart of thrust/system/cuda/detail/get_value.h):
// one element of device memory read back to the host.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/system/cdna4/detail/core.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class D, class T>
typename std::remove_const<T>::type get_value(const execution_policy<D>& exec, device_ptr<T> ptr) {
  typename std::remove_const<T>::type v;
  detail::throw_on_error(thrust_cdna4_read_back(&v, ptr.get(), sizeof(T), detail::stream_of(exec.derived())), "get_value");
  return v;
}
}}  // namespace system::cdna4
}  // namespace thrust
