// thrust::raw_reference_cast (thrust/detail/raw_reference_cast.h): the plain reference behind a
// device_reference; any other reference is returned as it is.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/functional.h>
#define THRUST_CDNA4_RRC_HD THRUST_CDNA4_HD
namespace thrust {
template <class T> THRUST_CDNA4_RRC_HD inline T& raw_reference_cast(T& r) { return r; }
template <class T> THRUST_CDNA4_HD inline T& raw_reference_cast(const device_reference<T>& r) { return *(&r).get(); }
}  // namespace thrust
