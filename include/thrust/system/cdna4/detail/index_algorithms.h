// Two entry points the small algorithm headers are written on: body(i) for every index of a
// range, and a reduction of load(i) over a range.  Kernel templates under hipcc
// (thrust/system/cuda/detail/parallel_for.h:70-174, reduce.h:152-669); under a host compiler a
// device range is a compile error that asks for hipcc.
#pragma once
#include <cstdint>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust { namespace system { namespace cdna4 { namespace detail {

template <class Policy, class Body>
void for_each_index(const Policy& exec, std::int64_t n, Body body, const char* what) {
  THRUST_CDNA4_NEEDS_HIPCC(Body);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, body);
  synchronize_optional(exec, what);
#else
  (void)exec; (void)n; (void)body; (void)what;
#endif
}

// op(init, load(0) (+) ... (+) load(n-1)); op associative and commutative; blocks for the value
template <class T, class Policy, class Load, class Op>
T reduce_index(const Policy& exec, std::int64_t n, Load load, T init, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(Load);
#if defined(__HIPCC__)
  return generic::transform_reduce(stream_of(exec), n, load, init, op);
#else
  (void)exec; (void)n; (void)load; (void)op;
  return init;
#endif
}

}}}}  // namespace thrust::system::cdna4::detail
