// for_each / transform / sequence / reduce / transform_reduce / count_if of the cdna4 system on
// contiguous device ranges with arbitrary functors.  With hipcc they instantiate the kernel
// templates of parallel_for.h; under a host compiler a device range is a compile error that
// says so (never a host fallback).
#pragma once
#include <cstdint>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/core.h>
#if defined(__HIPCC__)
#include <thrust/system/cdna4/detail/parallel_for.h>
#endif

namespace thrust { namespace system { namespace cdna4 { namespace detail {

#if defined(__HIPCC__)
#define THRUST_CDNA4_NEEDS_HIPCC(T) do { } while (0)
#else
template <class T> struct needs_hipcc { static constexpr bool value = sizeof(T) == 0; };
#define THRUST_CDNA4_NEEDS_HIPCC(T)                                                                        \
  static_assert(needs_hipcc<T>::value,                                                                     \
                "cdna4: algorithms with user functors on device ranges are kernel templates; compile this " \
                "translation unit with hipcc --offload-arch=gfx950")
#endif

#if defined(__HIPCC__)
template <class In, class F> struct for_each_body {
  In* p; F f;
  __device__ void operator()(std::int64_t i) { f(p[i]); }
};
template <class In, class Out, class F> struct transform1_body {
  const In* in; Out* out; F f;
  __device__ void operator()(std::int64_t i) { out[i] = f(in[i]); }
};
template <class In1, class In2, class Out, class F> struct transform2_body {
  const In1* a; const In2* b; Out* out; F f;
  __device__ void operator()(std::int64_t i) { out[i] = f(a[i], b[i]); }
};
template <class T> struct sequence_body {
  T* out; T init, step;
  __device__ void operator()(std::int64_t i) { out[i] = (T)(init + (T)i * step); }
};
template <class In, class F, class T> struct load_transform {
  const In* in; F f;
  __device__ T operator()(std::int64_t i) const { return (T)f(in[i]); }
};
#endif

template <class Policy, class In, class F>
void for_each_n(const Policy& exec, In* p, std::int64_t n, F f) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, for_each_body<In, F>{p, f});
  synchronize_optional(exec, "for_each: failed to synchronize");
#else
  (void)exec; (void)p; (void)n; (void)f;
#endif
}
template <class Policy, class In, class Out, class F>
void transform_n(const Policy& exec, const In* in, Out* out, std::int64_t n, F f) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, transform1_body<In, Out, F>{in, out, f});
  synchronize_optional(exec, "transform: failed to synchronize");
#else
  (void)exec; (void)in; (void)out; (void)n; (void)f;
#endif
}
template <class Policy, class In1, class In2, class Out, class F>
void transform_n(const Policy& exec, const In1* a, const In2* b, Out* out, std::int64_t n, F f) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, transform2_body<In1, In2, Out, F>{a, b, out, f});
  synchronize_optional(exec, "transform: failed to synchronize");
#else
  (void)exec; (void)a; (void)b; (void)out; (void)n; (void)f;
#endif
}
template <class Policy, class T>
void sequence_n(const Policy& exec, T* out, std::int64_t n, T init, T step) {
  THRUST_CDNA4_NEEDS_HIPCC(T);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, sequence_body<T>{out, init, step});
  synchronize_optional(exec, "sequence: failed to synchronize");
#else
  (void)exec; (void)out; (void)n; (void)init; (void)step;
#endif
}
template <class Policy, class In, class F, class T, class Op>
T transform_reduce_n(const Policy& exec, const In* in, std::int64_t n, F f, T init, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  return generic::transform_reduce(stream_of(exec), n, load_transform<In, F, T>{in, f}, init, op);
#else
  (void)exec; (void)in; (void)n; (void)f; (void)op;
  return init;
#endif
}

}}}}  // namespace thrust::system::cdna4::detail
