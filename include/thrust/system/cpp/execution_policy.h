// thrust::system::cpp / thrust::cpp (thrust/system/cpp/execution_policy.h): the host system of this
// build — sequential algorithms on host memory.  thrust::cpp::par is the policy object
// thrust::host also names; thrust::cpp::tag is the system tag of host iterators.
#pragma once
#include <thrust/execution_policy.h>
namespace thrust {
namespace system { namespace cpp {
static const detail::par_t par;
template <class Derived> using execution_policy = thrust::host_execution_policy<Derived>;
}}  // namespace system::cpp
namespace cpp {
using thrust::system::cpp::execution_policy;
using thrust::system::cpp::par;
using thrust::system::cpp::tag;
}  // namespace cpp
}  // namespace thrust
