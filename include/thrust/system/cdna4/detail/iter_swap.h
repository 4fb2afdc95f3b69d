// The cdna4 device system's iter_swap (the counterpart of thrust/system/cuda/detail/iter_swap.h): two
// elements of device memory exchanged from the host.
#pragma once
#include <thrust/system/cdna4/detail/assign_value.h>
#include <thrust/system/cdna4/detail/get_value.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class D, class T>
void iter_swap(const execution_policy<D>& exec, device_ptr<T> a, device_ptr<T> b) {
  const T va = get_value(exec, a), vb = get_value(exec, b);
  assign_value(exec, a, &vb);
  assign_value(exec, b, &va);
}
}}  // namespace system::cdna4
}  // namespace thrust
