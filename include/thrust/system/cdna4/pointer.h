// thrust::cdna4::pointer / reference (the counterpart of thrust/system/cuda/pointer.h): the device
// system's pointer is thrust::device_ptr, whose reference reads and writes single elements of device
// memory from the host.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/system/cdna4/detail/execution_policy.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class T> using pointer = thrust::device_ptr<T>;
template <class T> using reference = thrust::device_reference<T>;
template <class T> using universal_pointer = thrust::device_ptr<T>;
}}  // namespace system::cdna4
namespace cdna4 {
using thrust::system::cdna4::pointer;
using thrust::system::cdna4::reference;
using thrust::system::cdna4::universal_pointer;
}  // namespace cdna4
}  // namespace thrust
