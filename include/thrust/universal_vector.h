// thrust::universal_vector (thrust/universal_vector.h): a device_vector whose storage host code
// can address too (managed memory).  The algorithms treat it as a device range;
// raw_pointer_cast(v.data()) may be read and written on the host once device work on it is done.
#pragma once
#include <thrust/device_vector.h>
#include <thrust/universal_allocator.h>
namespace thrust {
template <class T, class Alloc = universal_allocator<T>> using universal_vector = device_vector<T, Alloc>;
}  // namespace thrust
