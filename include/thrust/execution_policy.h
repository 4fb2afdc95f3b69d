// thrust::device, thrust::host and the cdna4 stream policies (thrust/execution_policy.h:295, :344).
#pragma once
#include <thrust/system/cdna4/detail/core.h>
#include <thrust/detail/seq.h>

namespace thrust {
// Bases for user-defined policies and tags (thrust/execution_policy.h:63-, :171-): an algorithm
// called with a policy derived from device_execution_policy runs on the cdna4 system.
template <class Derived> using device_execution_policy = system::cdna4::execution_policy<Derived>;
template <class Derived> struct host_execution_policy : system::cpp::detail::par_t {};
namespace detail {
typedef system::cpp::detail::par_t host_t;
typedef system::cdna4::detail::par_t device_t;
}  // namespace detail
}  // namespace thrust
