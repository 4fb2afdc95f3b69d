// thrust::seq (thrust/detail/seq.h:34-52, thrust/execution_policy.h:347-384): the policy that runs
// an algorithm sequentially in the calling thread — on the host, or inside a kernel on a range
// that belongs to one thread.  The reference reaches its sequential system from device code the
// same way (thrust/system/cuda/detail/par_to_seq.h, cdp_dispatch.h:45-88).  The algorithms that
// take it are the __host__ __device__ loops of thrust/system/detail/sequential/; it is not
// derived from the device system's policy, so no kernel is ever launched for it.
#pragma once
#include <thrust/detail/hd.h>

namespace thrust {
namespace system { namespace detail { namespace sequential {
struct tag {};
template <class Derived> struct execution_policy {
  typedef tag tag_type;
};
}}}  // namespace system::detail::sequential
namespace detail {
struct seq_t : system::detail::sequential::execution_policy<seq_t> {
  THRUST_CDNA4_HD constexpr seq_t() {}
};
}  // namespace detail
// one object per translation unit and per side: device code refers to the device's copy
#if defined(__HIP_DEVICE_COMPILE__)
static const __device__ detail::seq_t seq;
#else
static const detail::seq_t seq;
#endif
}  // namespace thrust
