// for_each / transform / sequence / reduce / transform_reduce / count_if of the cdna4 system on
// contiguous device ranges with arbitrary functors.  With hipcc they instantiate the kernel
// templates of parallel_for.h; under a host compiler a device range is a compile error that
// says so (never a host fallback).
#pragma once
#include <cstdint>
#include <iterator>
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
  static_assert(::thrust::system::cdna4::detail::needs_hipcc<T>::value,                                     \
                "cdna4: algorithms with user functors on device ranges are kernel templates; compile this " \
                "translation unit with hipcc --offload-arch=gfx950")
#endif

// Stands for "no values" where keys-only and by-key forms share an implementation (merge, set
// operations): indexable, never read for its content.
struct no_values {
  THRUST_CDNA4_HD char operator[](std::int64_t) const { return 0; }
};

// In the bodies below an "iterator" is whatever detail::unwrap gives a kernel: a raw pointer or a
// fancy iterator over raw pointers, indexable on the device.
#if defined(__HIPCC__)
template <class It> struct value_of_it { typedef typename std::iterator_traits<It>::value_type type; };
template <class It, class F> struct for_each_body {
  It p; F f;
  __device__ void operator()(std::int64_t i) { f(p[i]); }
};
template <class In, class Out, class F> struct transform1_body {
  In in; Out out; F f;
  __device__ void operator()(std::int64_t i) { out[i] = f(in[i]); }
};
template <class In1, class In2, class Out, class F> struct transform2_body {
  In1 a; In2 b; Out out; F f;
  __device__ void operator()(std::int64_t i) { out[i] = f(a[i], b[i]); }
};
template <class Out, class T> struct sequence_body {
  Out out; T init, step;
  __device__ void operator()(std::int64_t i) { out[i] = at(i, std::is_arithmetic<T>()); }
  __device__ T at(std::int64_t i, std::true_type) const { return (T)(init + (T)i * step); }
  // a number-like class: init + step * i with the index as it is (thrust/system/detail/generic/sequence.inl:36-60)
  __device__ T at(std::int64_t i, std::false_type) const { return init + step * (std::size_t)i; }
};
template <class In, class F, class T> struct load_transform {
  In in; mutable F f;
  __device__ T operator()(std::int64_t i) const { return (T)f(in[i]); }
};
#endif

template <class Policy, class It, class F>
void apply_n(const Policy& exec, It p, std::int64_t n, F f) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, for_each_body<It, F>{p, f});
  synchronize_optional(exec, "for_each: failed to synchronize");
#else
  (void)exec; (void)p; (void)n; (void)f;
#endif
}
template <class Policy, class In, class Out, class F>
void transform_n(const Policy& exec, In in, Out out, std::int64_t n, F f) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, transform1_body<In, Out, F>{in, out, f});
  synchronize_optional(exec, "transform: failed to synchronize");
#else
  (void)exec; (void)in; (void)out; (void)n; (void)f;
#endif
}
template <class Policy, class In1, class In2, class Out, class F>
void transform_n(const Policy& exec, In1 a, In2 b, Out out, std::int64_t n, F f) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, transform2_body<In1, In2, Out, F>{a, b, out, f});
  synchronize_optional(exec, "transform: failed to synchronize");
#else
  (void)exec; (void)a; (void)b; (void)out; (void)n; (void)f;
#endif
}
template <class Policy, class Out, class T>
void sequence_n(const Policy& exec, Out out, std::int64_t n, T init, T step) {
  THRUST_CDNA4_NEEDS_HIPCC(T);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, sequence_body<Out, T>{out, init, step});
  synchronize_optional(exec, "sequence: failed to synchronize");
#else
  (void)exec; (void)out; (void)n; (void)init; (void)step;
#endif
}
template <class Policy, class In, class F, class T, class Op>
T transform_reduce_n(const Policy& exec, In in, std::int64_t n, F f, T init, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(F);
#if defined(__HIPCC__)
  return generic::transform_reduce(stream_of(exec), n, load_transform<In, F, T>{in, f}, init, op);
#else
  (void)exec; (void)in; (void)n; (void)f; (void)op;
  return init;
#endif
}

// ---- stable compaction (copy_if / remove_if / unique / unique_by_key / partition) -------
#if defined(__HIPCC__)
// keep in[i] when pred(in[i]) != NEGATE
template <class In, class Out, class Pred, bool NEGATE> struct keep_if_op {
  typedef typename value_of_it<In>::type item;
  static constexpr bool rejects = false;
  static constexpr int rows = sizeof(item) <= 4 ? 64 : sizeof(item) == 8 ? 32 : generic::select_rows(sizeof(item));  // 256 KiB tiles: see select_rows_of
  In in; Out out; mutable Pred pred;
  __device__ item load(std::int64_t i, bool& keep) const {
    const item x = in[i];
    keep = (bool)pred(x) != NEGATE;
    return x;
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
// keep in[i] when pred(stencil[i]) != NEGATE
template <class In, class S, class Out, class Pred, bool NEGATE> struct keep_if_stencil_op {
  typedef typename value_of_it<In>::type item;
  static constexpr bool rejects = false;
  In in; S stencil; Out out; mutable Pred pred;
  __device__ item load(std::int64_t i, bool& keep) const {
    keep = (bool)pred(stencil[i]) != NEGATE;
    return in[i];
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
// in[i] goes to out_true when pred(stencil[i]), else to out_false, both in order
template <class In, class S, class OutT, class OutF, class Pred> struct partition_op {
  typedef typename value_of_it<In>::type item;
  static constexpr bool rejects = true;
  In in; S stencil; OutT out_true; OutF out_false; mutable Pred pred;
  __device__ item load(std::int64_t i, bool& keep) const {
    keep = (bool)pred(stencil[i]);
    return in[i];
  }
  __device__ void store(const item& x, std::int64_t pos) const { out_true[pos] = x; }
  __device__ void store_rejected(const item& x, std::int64_t pos) const { out_false[pos] = x; }
};
// keep the first element of every run; element 0 compares with itself and is kept by index
template <class KIn, class KOut, class Eq> struct run_head_op {
  typedef typename value_of_it<KIn>::type item;
  static constexpr bool rejects = false;
  KIn keys; KOut out; mutable Eq eq;
  __device__ item load(std::int64_t i, bool& keep) const {
    const item cur = keys[i], prev = keys[i > 0 ? i - 1 : 0];
    keep = (i == 0) | !(bool)eq(prev, cur);
    return cur;
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
template <class KIn, class VIn, class KOut, class VOut, class Eq> struct run_head_by_key_op {
  typedef typename value_of_it<KIn>::type K;
  typedef typename value_of_it<VIn>::type V;
  struct item { K key; V value; };
  static constexpr bool rejects = false;
  static constexpr int rows = sizeof(item) == 8 ? 32 : generic::select_rows(sizeof(item));  // 256-byte tiles per thread: see select_rows_of
  KIn keys; VIn values; KOut kout; VOut vout; mutable Eq eq;
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
std::int64_t copy_flagged_n(const Policy& exec, In in, Out out, std::int64_t n, Pred pred) {
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
std::int64_t copy_flagged_n(const Policy& exec, In in, S stencil, Out out, std::int64_t n, Pred pred) {
  THRUST_CDNA4_NEEDS_HIPCC(Pred);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, keep_if_stencil_op<In, S, Out, Pred, NEGATE>{in, stencil, out, pred});
#else
  (void)exec; (void)in; (void)stencil; (void)out; (void)n; (void)pred;
  return 0;
#endif
}
// stable two-way split by pred(stencil[i]); returns the number that went to out_true
// a contiguous input is read through a pointer to const; any other iterator as it is
template <class T> inline const T* as_input(T* p) { return p; }
template <class It> inline It as_input(It it) { return it; }
template <class Policy, class In, class S, class OutT, class OutF, class Pred>
std::int64_t partition_copy_n(const Policy& exec, In in, S stencil, OutT out_true, OutF out_false, std::int64_t n, Pred pred) {
  THRUST_CDNA4_NEEDS_HIPCC(Pred);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, partition_op<In, S, OutT, OutF, Pred>{in, stencil, out_true, out_false, pred});
#else
  (void)exec; (void)in; (void)stencil; (void)out_true; (void)out_false; (void)n; (void)pred;
  return 0;
#endif
}
// out[0, count) = the first element of every run of equal elements; returns count
template <class Policy, class KIn, class KOut, class Eq>
std::int64_t unique_copy_n(const Policy& exec, KIn in, KOut out, std::int64_t n, Eq eq) {
  THRUST_CDNA4_NEEDS_HIPCC(Eq);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, run_head_op<KIn, KOut, Eq>{in, out, eq});
#else
  (void)exec; (void)in; (void)out; (void)n; (void)eq;
  return 0;
#endif
}
template <class Policy, class KIn, class VIn, class KOut, class VOut, class Eq>
std::int64_t unique_by_key_copy_n(const Policy& exec, KIn keys, VIn vals, KOut kout, VOut vout, std::int64_t n, Eq eq) {
  THRUST_CDNA4_NEEDS_HIPCC(Eq);
#if defined(__HIPCC__)
  return generic::select(stream_of(exec), n, run_head_by_key_op<KIn, VIn, KOut, VOut, Eq>{keys, vals, kout, vout, eq});
#else
  (void)exec; (void)keys; (void)vals; (void)kout; (void)vout; (void)n; (void)eq;
  return 0;
#endif
}

// ---- adjacent_difference, vectorised binary searches ------------------------------------
#if defined(__HIPCC__)
template <class In, class Out, class Op> struct adjacent_difference_body {
  In in; Out out; Op op;
  __device__ void operator()(std::int64_t i) {
    typedef typename value_of_it<In>::type T;
    const T cur = in[i];
    if (i == 0) out[i] = cur;
    else out[i] = op(cur, (T)in[i - 1]);
  }
};
// MODE 0: first position whose element is not less than the value (lower bound); 1: first
// position whose element is greater (upper bound); 2: whether an equivalent element exists
template <int MODE, class Hay, class Needles, class Out, class Comp> struct binary_search_body {
  Hay hay; std::int64_t count; Needles needles; Out out; Comp comp;
  __device__ void operator()(std::int64_t i) {
    const auto v = needles[i];
    std::int64_t lo = 0, len = count;
    while (len > 0) {
      const std::int64_t half = len >> 1;
      const bool right = MODE == 1 ? !(bool)comp(v, hay[lo + half]) : (bool)comp(hay[lo + half], v);
      lo = right ? lo + half + 1 : lo;
      len = right ? len - half - 1 : half;
    }
    if (MODE == 2) out[i] = lo < count && !(bool)comp(v, hay[lo]);
    else out[i] = lo;
  }
};
#endif
template <class Policy, class In, class Out, class Op>
void adjacent_difference_n(const Policy& exec, In in, Out out, std::int64_t n, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(Op);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, adjacent_difference_body<In, Out, Op>{in, out, op});
  synchronize_optional(exec, "adjacent_difference: failed to synchronize");
#else
  (void)exec; (void)in; (void)out; (void)n; (void)op;
#endif
}
template <int MODE, class Policy, class Hay, class Needles, class Out, class Comp>
void binary_search_n(const Policy& exec, Hay hay, std::int64_t count, Needles needles, Out out, std::int64_t n, Comp comp) {
  THRUST_CDNA4_NEEDS_HIPCC(Comp);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, binary_search_body<MODE, Hay, Needles, Out, Comp>{hay, count, needles, out, comp});
  synchronize_optional(exec, "binary search: failed to synchronize");
#else
  (void)exec; (void)hay; (void)count; (void)needles; (void)out; (void)n; (void)comp;
#endif
}

// out[i] = in[index[i]]
#if defined(__HIPCC__)
template <class In, class Index, class Out> struct gather_body {
  In in; Index index; Out out;
  __device__ void operator()(std::int64_t i) { out[i] = in[index[i]]; }
};
#endif
template <class Policy, class In, class Index, class Out>
void gather_n(const Policy& exec, In in, Index index, Out out, std::int64_t n) {
  THRUST_CDNA4_NEEDS_HIPCC(In);
#if defined(__HIPCC__)
  generic::parallel_for(stream_of(exec), n, gather_body<In, Index, Out>{in, index, out});
  synchronize_optional(exec, "gather: failed to synchronize");
#else
  (void)exec; (void)in; (void)index; (void)out; (void)n;
#endif
}

// ---- fancy iterators around the C-ABI algorithms (sort, scan, by-key) --------------------
// Those kernels read and write contiguous arrays.  A raw pointer passes through; any other
// iterator is read into (input) or written from (output) a pool temporary by one generic kernel.
template <class T, class It, bool RAW = std::is_pointer<It>::value> class contiguous_input;
template <class T, class It> class contiguous_input<T, It, true> {
 public:
  template <class Policy> contiguous_input(const Policy&, It it, std::int64_t) : p_(it) {
    static_assert(std::is_same<T, typename std::remove_const<typename std::remove_pointer<It>::type>::type>::value,
                  "cdna4: the element type of this range must match the algorithm's");
  }
  const T* data() const { return p_; }
 private:
  const T* p_;
};
template <class T, class It> class contiguous_input<T, It, false> {
 public:
  template <class Policy> contiguous_input(const Policy& exec, It it, std::int64_t n)
      : tmp_((std::size_t)(n > 0 ? n : 0) * sizeof(T), stream_of(exec)) {
    THRUST_CDNA4_NEEDS_HIPCC(It);
#if defined(__HIPCC__)
    generic::parallel_for(stream_of(exec), n, transform1_body<It, T*, thrust::identity<T>>{it, static_cast<T*>(tmp_.data()), thrust::identity<T>()});
#else
    (void)it;
#endif
  }
  const T* data() const { return static_cast<const T*>(tmp_.data()); }
 private:
  temporary_storage tmp_;
};
template <class T, class It, bool RAW = std::is_pointer<It>::value> class contiguous_output;
template <class T, class It> class contiguous_output<T, It, true> {
 public:
  template <class Policy> contiguous_output(const Policy&, It it, std::int64_t) : p_(it) {
    static_assert(std::is_same<T, typename std::remove_pointer<It>::type>::value,
                  "cdna4: the element type of the output range must match the algorithm's");
  }
  T* data() const { return p_; }
  template <class Policy> void flush(const Policy&, std::int64_t) {}
 private:
  T* p_;
};
template <class T, class It> class contiguous_output<T, It, false> {
 public:
  template <class Policy> contiguous_output(const Policy& exec, It it, std::int64_t n)
      : it_(it), tmp_((std::size_t)(n > 0 ? n : 0) * sizeof(T), stream_of(exec)) {}
  T* data() const { return static_cast<T*>(tmp_.data()); }
  // the first count elements go to the iterator
  template <class Policy> void flush(const Policy& exec, std::int64_t count) {
    THRUST_CDNA4_NEEDS_HIPCC(It);
#if defined(__HIPCC__)
    generic::parallel_for(stream_of(exec), count, transform1_body<const T*, It, thrust::identity<T>>{data(), it_, thrust::identity<T>()});
    synchronize_optional(exec, "output: failed to synchronize");
#else
    (void)exec; (void)count;
#endif
  }
 private:
  It it_;
  temporary_storage tmp_;
};

// the address behind a raw pointer (only raw pointers can alias an output range)
template <class T> inline const void* address_of(T* p) { return p; }
template <class It> inline const void* address_of(It) { return nullptr; }

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
