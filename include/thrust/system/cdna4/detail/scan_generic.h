// inclusive_scan / exclusive_scan / *_scan_by_key / reduce_by_key of the cdna4 system for
// everything the precompiled kernels behind the C ABI do not cover: user-defined operators and
// predicates, accumulator types that differ from the element type, struct elements, fancy
// iterators read in place, more than 2^32 - 1 elements.  The operations below run on the
// one-pass prefix engine of scan_engine.h; they exist when the translation unit is compiled by
// hipcc, and are a compile error that says so under a host compiler.
//
// Accumulator types follow the reference: the input's value type for inclusive_scan
// (thrust/system/cuda/detail/scan.h:63), the type of `init` for exclusive_scan (:142-154), and
// likewise for the by-key forms (scan_by_key.h:69-282); reduce_by_key accumulates in the value
// input's type.  An element is converted to the accumulator type when it is loaded and every
// result of the operator is converted back to it, as `accum = op(accum, x)` does in the
// sequential system (thrust/system/detail/sequential/scan.h:47-114).
#pragma once
#include <cstdint>
#include <thrust/system/cdna4/detail/generic_algorithms.h>
#if defined(__HIPCC__)
#include <thrust/system/cdna4/detail/scan_engine.h>
#endif

namespace thrust { namespace system { namespace cdna4 { namespace detail {

#if defined(__HIPCC__)
template <class In, class Out, class Acc, class Op, bool EXCLUSIVE>
struct scan_body {
  typedef Acc acc;
  In in; Out out; Acc init; mutable Op op;
  __device__ Acc load(std::int64_t i) const { return static_cast<Acc>(in[i]); }
  __device__ Acc combine(const Acc& a, const Acc& b) const { return static_cast<Acc>(op(a, b)); }
  __device__ void store(std::int64_t i, bool has_before, const Acc& before, const Acc& upto) const {
    if (EXCLUSIVE) out[i] = has_before ? static_cast<Acc>(op(init, before)) : init;
    else out[i] = upto;
  }
};

// (segment heads seen, value of the open segment); C counts heads (scan_by_key only asks whether
// there are any, reduce_by_key uses the count as the output position)
template <class C, class V>
struct seg_acc {
  C c;
  V v;
};

template <class KIn, class VIn, class Out, class V, class Pred, class Op, bool EXCLUSIVE>
struct scan_by_key_body {
  typedef seg_acc<unsigned, V> acc;
  KIn keys; VIn vals; Out out; V init; mutable Pred pred; mutable Op op;
  // a head is an element whose key does not continue its predecessor's segment
  // (thrust/system/detail/sequential/scan_by_key.h:63-83: pred(previous key, key))
  __device__ acc load(std::int64_t i) const {
    const bool head = (i == 0) | !pred(keys[i > 0 ? i - 1 : 0], keys[i]);  // no branch around the loads
    return acc{head ? 1u : 0u, static_cast<V>(vals[i])};
  }
  __device__ acc combine(const acc& a, const acc& b) const {
    return acc{(a.c | b.c) ? 1u : 0u, b.c ? b.v : static_cast<V>(op(a.v, b.v))};
  }
  __device__ void store(std::int64_t i, bool has_before, const acc& before, const acc& upto) const {
    if (!EXCLUSIVE) {
      out[i] = upto.v;
    } else {
      // init restarts at every head (sequential/scan_by_key.h:95-140)
      const bool head = (i == 0) | !pred(keys[i > 0 ? i - 1 : 0], keys[i]);  // no branch around the loads
      out[i] = (head || !has_before) ? init : static_cast<V>(op(init, before.v));
    }
  }
};

template <class C, class KIn, class VIn, class KOut, class VOut, class V, class Pred, class Op>
struct reduce_by_key_body {
  typedef seg_acc<C, V> acc;
  KIn keys; VIn vals; KOut kout; VOut vout; long long* num_runs; std::int64_t n; mutable Pred pred; mutable Op op;
  __device__ acc load(std::int64_t i) const {
    const bool head = (i == 0) | !pred(keys[i > 0 ? i - 1 : 0], keys[i]);  // no branch around the loads
    return acc{(C)(head ? 1 : 0), static_cast<V>(vals[i])};
  }
  __device__ acc combine(const acc& a, const acc& b) const {
    return acc{(C)(a.c + b.c), b.c ? b.v : static_cast<V>(op(a.v, b.v))};
  }
  // a head writes its key and closes the run before it; the last element closes the last run
  // (thrust/system/detail/sequential/reduce_by_key.h:58-92)
  __device__ void store(std::int64_t i, bool has_before, const acc& before, const acc& upto) const {
    const bool head = !has_before || upto.c != before.c;
    if (head) {
      kout[(std::int64_t)upto.c - 1] = keys[i];
      if (has_before) vout[(std::int64_t)before.c - 1] = before.v;
    }
    if (i == n - 1) {
      vout[(std::int64_t)upto.c - 1] = upto.v;
      *num_runs = (long long)upto.c;
    }
  }
};
#endif

template <bool EXCLUSIVE, class Acc, class Policy, class In, class Out, class Op>
void generic_scan(const Policy& exec, In in, Out out, std::int64_t n, Acc init, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(Op);
#if defined(__HIPCC__)
  generic::scan_engine(stream_of(exec), n, scan_body<In, Out, Acc, Op, EXCLUSIVE>{in, out, init, op});
  synchronize_optional(exec, "scan: failed to synchronize");
#else
  (void)exec; (void)in; (void)out; (void)n; (void)init; (void)op;
#endif
}

// An output written over the KEYS (testing/scan_by_key.inclusive.cu:325-334 does it): the engine
// reads the key before an element from memory, some of them after other elements' results have
// been stored.  Keys and output that are both given by raw pointers and share a byte are told apart
// here, and the keys are then read from a copy; ranges behind other iterators cannot be compared.
template <class KIn, class Out>
inline std::size_t keys_to_set_aside(KIn, Out, std::int64_t) { return 0; }
template <class K, class O>
inline std::size_t keys_to_set_aside(K* keys, O* out, std::int64_t n) {
  const char* k = reinterpret_cast<const char*>(keys);
  const char* o = reinterpret_cast<const char*>(out);
  const bool overlap = n > 0 && k < o + n * (std::int64_t)sizeof(O) && o < k + n * (std::int64_t)sizeof(K);
  return overlap ? (std::size_t)n * sizeof(K) : 0;
}
template <class KIn>
inline KIn keys_set_aside(KIn keys, void*, std::size_t, void*) { return keys; }
template <class K>
inline K* keys_set_aside(K* keys, void* copy, std::size_t bytes, void* stream) {
  if (!bytes) return keys;
  throw_on_error(thrust_cdna4_memcpy_dtod(copy, keys, bytes, stream), "by key: setting the keys aside");
  return static_cast<K*>(copy);
}

template <bool EXCLUSIVE, class V, class Policy, class KIn, class VIn, class Out, class Pred, class Op>
void generic_scan_by_key(const Policy& exec, KIn keys, VIn vals, Out out, std::int64_t n, V init, Pred pred, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(Op);
#if defined(__HIPCC__)
  const std::size_t aside = keys_to_set_aside(keys, out, n);
  temporary_storage hold(aside, exec);
  keys = keys_set_aside(keys, hold.data(), aside, stream_of(exec));
  generic::scan_engine(stream_of(exec), n, scan_by_key_body<KIn, VIn, Out, V, Pred, Op, EXCLUSIVE>{keys, vals, out, init, pred, op});
  synchronize_optional(exec, "scan_by_key: failed to synchronize");
#else
  (void)exec; (void)keys; (void)vals; (void)out; (void)n; (void)init; (void)pred; (void)op;
#endif
}

// Returns the number of runs; blocks until it is known, as the reference does
// (thrust/system/cuda/detail/reduce_by_key.h:1049-1052).
template <class V, class Policy, class KIn, class VIn, class KOut, class VOut, class Pred, class Op>
std::int64_t generic_reduce_by_key(const Policy& exec, KIn keys, VIn vals, KOut kout, VOut vout, std::int64_t n, Pred pred, Op op) {
  THRUST_CDNA4_NEEDS_HIPCC(Op);
#if defined(__HIPCC__)
  if (n <= 0) return 0;
  const std::size_t aside = keys_to_set_aside(keys, kout, n) ? keys_to_set_aside(keys, kout, n) : keys_to_set_aside(keys, vout, n);
  temporary_storage hold(aside, exec);
  keys = keys_set_aside(keys, hold.data(), aside, stream_of(exec));
  temporary_storage tmp(256, exec);
  long long* d_runs = static_cast<long long*>(tmp.data());
  if (n < (std::int64_t(1) << 32))
    generic::scan_engine(stream_of(exec), n, reduce_by_key_body<unsigned, KIn, VIn, KOut, VOut, V, Pred, Op>{keys, vals, kout, vout, d_runs, n, pred, op});
  else
    generic::scan_engine(stream_of(exec), n, reduce_by_key_body<long long, KIn, VIn, KOut, VOut, V, Pred, Op>{keys, vals, kout, vout, d_runs, n, pred, op});
  long long runs = 0;
  throw_on_error(thrust_cdna4_read_back(&runs, d_runs, sizeof(runs), stream_of(exec)), "reduce_by_key: read run count");
  return (std::int64_t)runs;
#else
  (void)exec; (void)keys; (void)vals; (void)kout; (void)vout; (void)n; (void)pred; (void)op;
  return 0;
#endif
}

}}}}  // namespace thrust::system::cdna4::detail
