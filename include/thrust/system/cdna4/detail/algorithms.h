// Device algorithms of the cdna4 system on raw device pointers: each one classifies its
// arguments (arithmetic element type, built-in functor), runs the two-phase C-ABI protocol
// with algorithm-scoped temporary storage from the cached allocator, and synchronises the
// stream unless the policy says otherwise.  Mirrors
//   thrust/system/cuda/detail/sort.h:306-380, :431-484      (radix_sort, smart_sort)
//   thrust/system/cuda/detail/scan.h:57-204                 (inclusive/exclusive_scan_n_impl)
//   thrust/system/cuda/detail/scan_by_key.h:69-282
//   thrust/system/cuda/detail/reduce_by_key.h:979-1102      (reduce_by_key_dispatch)
#pragma once
#include <cstdint>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/core.h>
#if defined(__HIPCC__)
#include <thrust/system/cdna4/detail/merge_sort.h>
#endif

namespace thrust { namespace system { namespace cdna4 { namespace detail {

// Arithmetic keys under thrust::less / thrust::greater take the radix kernels behind the C ABI
// (thrust/system/cuda/detail/sort.h:389-395, can_use_primitive_sort); everything else is a
// comparison sort with kernel templates, which exist only when this header is compiled by hipcc.
template <class K, class Compare>
struct use_radix_sort : std::integral_constant<bool, dtype_of<K>::supported && (order_code<Compare>::value >= 0)> {};

template <class Policy, class K, class Compare>
void sort_keys_impl(const Policy& exec, K* keys, std::int64_t n, Compare, std::true_type) {
  void* s = stream_of(exec);
  std::size_t bytes = 0;
  throw_on_error(thrust_cdna4_sort_keys(nullptr, &bytes, dtype_of<K>::value, keys, n, order_code<Compare>::value, s),
                 "sort: temporary storage query");
  temporary_storage tmp(bytes, exec);
  throw_on_error(thrust_cdna4_sort_keys(tmp.data(), &bytes, dtype_of<K>::value, keys, n, order_code<Compare>::value, s),
                 "sort: launch");
  // a synchronous call waits here and learns whether every wait inside the sort ended
  // (thrust/system/cuda/detail/util.h:207-292); par_nosync leaves that to the caller
  if (must_sync(exec)) throw_on_error(thrust_cdna4_sort_status(tmp.data(), n, s), "sort: a wait inside the sort did not end");
}
template <class Policy, class K, class Compare>
void sort_keys_impl(const Policy& exec, K* keys, std::int64_t n, Compare comp, std::false_type) {
#if defined(__HIPCC__)
  merge::stable_sort(stream_of(exec), keys, static_cast<merge::no_value*>(nullptr), n, comp);
#else
  static_assert(sizeof(K) == 0,
                "cdna4 sort: a custom comparator or non-arithmetic key needs the comparison-sort kernel templates; "
                "compile this translation unit with hipcc --offload-arch=gfx950");
  (void)exec; (void)keys; (void)n; (void)comp;
#endif
}

template <class Policy, class K, class Compare>
void sort_keys(const Policy& exec, K* keys, std::int64_t n, Compare comp) {
  if (n <= 0) return;  // thrust/system/cuda/detail/sort.h:140-143
  sort_keys_impl(exec, keys, n, comp, use_radix_sort<K, Compare>());
  synchronize_optional(exec, "sort: failed to synchronize");
}

template <class Policy, class K, class V, class Compare>
void sort_pairs_impl(const Policy& exec, K* keys, V* values, std::int64_t n, Compare, std::true_type) {
  void* s = stream_of(exec);
  std::size_t bytes = 0;
  throw_on_error(thrust_cdna4_sort_pairs(nullptr, &bytes, dtype_of<K>::value, keys, (int)sizeof(V), values, n,
                                         order_code<Compare>::value, s), "sort_by_key: temporary storage query");
  temporary_storage tmp(bytes, exec);
  throw_on_error(thrust_cdna4_sort_pairs(tmp.data(), &bytes, dtype_of<K>::value, keys, (int)sizeof(V), values, n,
                                         order_code<Compare>::value, s), "sort_by_key: launch");
  if (must_sync(exec)) throw_on_error(thrust_cdna4_sort_status(tmp.data(), n, s), "sort_by_key: a wait inside the sort did not end");
}
template <class Policy, class K, class V, class Compare>
void sort_pairs_impl(const Policy& exec, K* keys, V* values, std::int64_t n, Compare comp, std::false_type) {
#if defined(__HIPCC__)
  merge::stable_sort(stream_of(exec), keys, values, n, comp);
#else
  static_assert(sizeof(K) == 0,
                "cdna4 sort_by_key: a custom comparator, non-arithmetic key or value wider than 8 bytes needs the "
                "comparison-sort kernel templates; compile this translation unit with hipcc --offload-arch=gfx950");
  (void)exec; (void)keys; (void)values; (void)n; (void)comp;
#endif
}

template <class Policy, class K, class V, class Compare>
void sort_pairs(const Policy& exec, K* keys, V* values, std::int64_t n, Compare comp) {
  static_assert(thrust::detail::is_bytewise_movable<V>::value, "cdna4 sort_by_key: values must be movable as bytes");
  if (n <= 0) return;
  constexpr bool radix_value = sizeof(V) == 1 || sizeof(V) == 2 || sizeof(V) == 4 || sizeof(V) == 8;
  sort_pairs_impl(exec, keys, values, n, comp,
                  std::integral_constant<bool, use_radix_sort<K, Compare>::value && radix_value>());
  synchronize_optional(exec, "sort_by_key: failed to synchronize");
}

template <class Policy, class T, class Op>
void scan(const Policy& exec, const T* in, T* out, std::int64_t n, bool exclusive, const T* init, Op) {
  static_assert(dtype_of<T>::supported, "cdna4 scan: elements must be an arithmetic type");
  static_assert(op_code<Op>::value >= 0, "cdna4 scan: only plus / multiplies / maximum / minimum have a kernel");
  if (n <= 0) return;
  void* s = stream_of(exec);
  std::size_t bytes = 0;
  throw_on_error(thrust_cdna4_scan(nullptr, &bytes, dtype_of<T>::value, op_code<Op>::value, exclusive, in, out, n, init, s),
                 "scan: temporary storage query");
  temporary_storage tmp(bytes, exec);
  throw_on_error(thrust_cdna4_scan(tmp.data(), &bytes, dtype_of<T>::value, op_code<Op>::value, exclusive, in, out, n, init, s),
                 "scan: launch");
  synchronize_optional(exec, "scan: failed to synchronize");
}

template <class Policy, class K, class T, class Pred, class Op>
void scan_by_key(const Policy& exec, const K* keys, const T* in, T* out, std::int64_t n, bool exclusive,
                 const T* init, Pred, Op) {
  static_assert(dtype_of<K>::supported && dtype_of<T>::supported, "cdna4 scan_by_key: arithmetic keys and values");
  static_assert(is_equal_to<Pred>::value, "cdna4 scan_by_key: only thrust::equal_to has a kernel");
  static_assert(op_code<Op>::value >= 0, "cdna4 scan_by_key: only plus / multiplies / maximum / minimum have a kernel");
  if (n <= 0) return;  // thrust/system/cuda/detail/scan_by_key.h:78-81
  void* s = stream_of(exec);
  std::size_t bytes = 0;
  throw_on_error(thrust_cdna4_scan_by_key(nullptr, &bytes, dtype_of<K>::value, dtype_of<T>::value, op_code<Op>::value,
                                          exclusive, keys, in, out, n, init, s), "scan_by_key: temporary storage query");
  temporary_storage tmp(bytes, exec);
  throw_on_error(thrust_cdna4_scan_by_key(tmp.data(), &bytes, dtype_of<K>::value, dtype_of<T>::value, op_code<Op>::value,
                                          exclusive, keys, in, out, n, init, s), "scan_by_key: launch");
  synchronize_optional(exec, "scan_by_key: failed to synchronize");
}

// Returns the number of runs.  Always synchronises: the count is read back from the device
// (thrust/system/cuda/detail/reduce_by_key.h:1049-1052).
template <class Policy, class K, class T, class Pred, class Op>
std::int64_t reduce_by_key(const Policy& exec, const K* keys, const T* vals, K* keys_out, T* vals_out,
                           std::int64_t n, Pred, Op) {
  static_assert(dtype_of<K>::supported && dtype_of<T>::supported, "cdna4 reduce_by_key: arithmetic keys and values");
  static_assert(is_equal_to<Pred>::value, "cdna4 reduce_by_key: only thrust::equal_to has a kernel");
  static_assert(op_code<Op>::value >= 0, "cdna4 reduce_by_key: only plus / multiplies / maximum / minimum have a kernel");
  if (n <= 0) return 0;  // thrust/system/cuda/detail/reduce_by_key.h:993-996
  void* s = stream_of(exec);
  std::size_t bytes = 0;
  throw_on_error(thrust_cdna4_reduce_by_key(nullptr, &bytes, dtype_of<K>::value, dtype_of<T>::value, op_code<Op>::value,
                                            keys, vals, keys_out, vals_out, nullptr, n, s),
                 "reduce_by_key: temporary storage query");
  temporary_storage tmp(bytes + 256, exec);  // + the run counter
  std::int64_t* d_runs = reinterpret_cast<std::int64_t*>(static_cast<char*>(tmp.data()) + bytes);
  throw_on_error(thrust_cdna4_reduce_by_key(tmp.data(), &bytes, dtype_of<K>::value, dtype_of<T>::value, op_code<Op>::value,
                                            keys, vals, keys_out, vals_out, d_runs, n, s), "reduce_by_key: launch");
  std::int64_t runs = 0;
  throw_on_error(thrust_cdna4_read_back(&runs, d_runs, sizeof(runs), s), "reduce_by_key: read run count");
  return runs;
}

}}}}  // namespace thrust::system::cdna4::detail
