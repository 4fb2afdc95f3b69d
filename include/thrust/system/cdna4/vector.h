// thrust::cdna4::vector / universal_vector (the counterpart of thrust/system/cuda/vector.h): the
// device system's vector is thrust::device_vector.
#pragma once
#include <thrust/device_vector.h>
#include <thrust/system/cdna4/memory.h>
#include <thrust/universal_vector.h>
namespace thrust {
namespace system { namespace cdna4 {
template <class T, class Allocator = thrust::device_allocator<T>> using vector = thrust::device_vector<T, Allocator>;
template <class T> using universal_vector = thrust::universal_vector<T>;
}}  // namespace system::cdna4
namespace cdna4 {
using thrust::system::cdna4::universal_vector;
using thrust::system::cdna4::vector;
}  // namespace cdna4
}  // namespace thrust
