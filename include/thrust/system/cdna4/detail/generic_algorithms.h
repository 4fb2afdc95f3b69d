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

// ---- stable compaction (copy_if / remove_if / unique / unique_by_key) ------------------
#if defined(__HIPCC__)
// keep in[i] when pred(in[i]) != NEGATE
template <class In, class Out, class Pred, bool NEGATE> struct keep_if_op {
  typedef In item;
  static constexpr bool rejects = false;
  const In* in; Out* out; Pred pred;
  __device__ item load(std::int64_t i, bool& keep) const {
    const In x = in[i];
    keep = (bool)pred(x) != NEGATE;
    return x;
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
// keep in[i] when pred(stencil[i]) != NEGATE
template <class In, class S, class Out, class Pred, bool NEGATE> struct keep_if_stencil_op {
  typedef In item;
  static constexpr bool rejects = false;
  const In* in; const S* stencil; Out* out; Pred pred;
  __device__ item load(std::int64_t i, bool& keep) const {
    keep = (bool)pred(stencil[i]) != NEGATE;
    return in[i];
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
// in[i] goes to out_true when pred(stencil[i]), else to out_false, both in order
template <class In, class S, class OutT, class OutF, class Pred> struct partition_op {
  typedef In item;
  static constexpr bool rejects = true;
  const In* in; const S* stencil; OutT* out_true; OutF* out_false; Pred pred;
  __device__ item load(std::int64_t i, bool& keep) const {
    keep = (bool)pred(stencil[i]);
    return in[i];
  }
  __device__ void store(const item& x, std::int64_t pos) const { out_true[pos] = x; }
  __device__ void store_rejected(const item& x, std::int64_t pos) const { out_false[pos] = x; }
};
// keep the first element of every run; element 0 compares with itself and is kept by index
template <class K, class KOut, class Eq> struct run_head_op {
  typedef K item;
  static constexpr bool rejects = false;
  const K* keys; KOut* out; Eq eq;
  __device__ item load(std::int64_t i, bool& keep) const {
    const K cur = keys[i], prev = keys[i > 0 ? i - 1 : 0];
    keep = (i == 0) | !(bool)eq(prev, cur);
    return cur;
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
template <class K, class V, class KOut, class VOut, class Eq> struct run_head_by_key_op {
  struct item { K key; V value; };
  static constexpr bool rejects = false;
  const K* keys; const V* values; KOut* kout; VOut* vout; Eq eq;
  __device__ item load(std::int64_t i, bool& keep) const {
    const K cur = keys[i], prev = keys[i > 0 ? i - 1 : 0];
    keep = (i == 0) | !(bool)eq(prev, cur);
    return item{cur, values[i]};
  }
  __device__ void store(const item& x, std::int64_t pos) const { kout[pos] = x.key; vout[pos] = x.value; }
};
#endif

// out[0, count) = the in[i] with pred(in[i]) != NEGATE, in order; returns count
template <bool NEGATE, class Policy, class In, class Out, class Pred>
std::int64_t copy_flagged_n(const Policy& exec, const In* in, Out* out, std::int64_t n, Pred pred) {
  THRUST_CDNA4_NEEDS_HIPCC(Pred);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, keep_if_op<In, Out, Pred, NEGATE>{in, out, pred});
#else
  (void)exec; (void)in; (void)out; (void)n; (void)pred;
  return 0;
#endif
}
// the same with the predicate applied to stencil[i]
template <bool NEGATE, class Policy, class In, class S, class Out, class Pred>
std::int64_t copy_flagged_n(const Policy& exec, const In* in, const S* stencil, Out* out, std::int64_t n, Pred pred) {
  THRUST_CDNA4_NEEDS_HIPCC(Pred);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, keep_if_stencil_op<In, S, Out, Pred, NEGATE>{in, stencil, out, pred});
#else
  (void)exec; (void)in; (void)stencil; (void)out; (void)n; (void)pred;
  return 0;
#endif
}
// stable two-way split by pred(stencil[i]); returns the number that went to out_true
template <class Policy, class In, class S, class OutT, class OutF, class Pred>
std::int64_t partition_copy_n(const Policy& exec, const In* in, const S* stencil, OutT* out_true, OutF* out_false, std::int64_t n, Pred pred) {
  THRUST_CDNA4_NEEDS_HIPCC(Pred);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, partition_op<In, S, OutT, OutF, Pred>{in, stencil, out_true, out_false, pred});
#else
  (void)exec; (void)in; (void)stencil; (void)out_true; (void)out_false; (void)n; (void)pred;
  return 0;
#endif
}
// out[0, count) = the first element of every run of equal elements; returns count
template <class Policy, class K, class KOut, class Eq>
std::int64_t unique_copy_n(const Policy& exec, const K* in, KOut* out, std::int64_t n, Eq eq) {
  THRUST_CDNA4_NEEDS_HIPCC(Eq);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, run_head_op<K, KOut, Eq>{in, out, eq});
#else
  (void)exec; (void)in; (void)out; (void)n; (void)eq;
  return 0;
#endif
}
template <class Policy, class K, class V, class KOut, class VOut, class Eq>
std::int64_t unique_by_key_copy_n(const Policy& exec, const K* keys, const V* vals, KOut* kout, VOut* vout, std::int64_t n, Eq eq) {
  THRUST_CDNA4_NEEDS_HIPCC(Eq);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, run_head_by_key_op<K, V, KOut, VOut, Eq>{keys, vals, kout, vout, eq});
#else
  (void)exec; (void)keys; (void)vals; (void)kout; (void)vout; (void)n; (void)eq;
  return 0;
#endif
}

// A device copy of [p, p + n) from the pool, for the in-place variants (the compaction reads its
// whole input while other tiles already write the front of the output).
template <class T>
class scratch_copy {
 public:
  scratch_copy(const T* p, std::int64_t n, void* stream) : tmp_((std::size_t)n * sizeof(T), stream) {
    if (n > 0) throw_on_error(thrust_cdna4_memcpy_dtod(tmp_.data(), p, (std::size_t)n * sizeof(T), stream), "temporary copy");
  }
  const T* data() const { return static_cast<const T*>(tmp_.data()); }
 private:
  temporary_storage tmp_;
};

}}}}  // namespace thrust::system::cdna4::detail
