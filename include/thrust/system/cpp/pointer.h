// thrust::cpp::pointer / reference (thrust/system/cpp/pointer.h): pointers into host memory are
// raw pointers in this build.
#pragma once
#include <thrust/system/cpp/execution_policy.h>
namespace thrust {
namespace system { namespace cpp {
template <class T> using pointer = T*;
template <class T> using reference = T&;
}}  // namespace system::cpp
namespace cpp {
using thrust::system::cpp::pointer;
using thrust::system::cpp::reference;
}  // namespace cpp
}  // namespace thrust
