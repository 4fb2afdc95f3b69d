// The cdna4 device system's partition (the counterpart of thrust/system/cuda/detail/partition.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/partition.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/partition.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// ---- device
template <class D, class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> stable_partition_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, St stencil,
                                       OutT out_true, OutF out_false, Pred pred) {
  typedef typename thrust::detail::value_of<In>::type V;
  typedef typename thrust::detail::value_of<St>::type S;
  const std::int64_t n = (std::int64_t)(last - first);
  const std::int64_t c = system::cdna4::detail::partition_copy_n(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(stencil),
                                                                 thrust::detail::unwrap(out_true), thrust::detail::unwrap(out_false), n, pred);
  return thrust::make_pair(out_true + c, out_false + (n - c));
}
template <class D, class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> stable_partition_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, OutT out_true, OutF out_false, Pred pred) {
  return stable_partition_copy(exec, first, last, first, out_true, out_false, pred);
}
namespace detail {
// In place over a range that is no array (a zip of arrays, say): the elements are gathered into a
// temporary, partitioned from there into the range and a second temporary, and the rejected ones
// copied behind the accepted.  STENCIL_IS_INPUT: the predicate reads the elements themselves.
template <bool STENCIL_IS_INPUT, class Policy, class It, class St, class Pred>
It stable_partition_gathered(const Policy& exec, It first, It last, St stencil, Pred pred) {
  typedef typename thrust::detail::value_of<It>::type V;
  const std::int64_t n = (std::int64_t)(last - first);
  if (n <= 0) return first;
  temporary_storage gathered((std::size_t)n * sizeof(V), exec), rejected((std::size_t)n * sizeof(V), exec);
  V* in = static_cast<V*>(gathered.data());
  V* rej = static_cast<V*>(rejected.data());
  thrust::copy(exec, first, last, thrust::device_ptr<V>(in));
  std::int64_t c;
  if constexpr (STENCIL_IS_INPUT) c = partition_copy_n(exec, (const V*)in, (const V*)in, thrust::detail::unwrap(first), rej, n, pred);
  else c = partition_copy_n(exec, (const V*)in, as_input(thrust::detail::unwrap(stencil)), thrust::detail::unwrap(first), rej, n, pred);
  thrust::copy(exec, thrust::device_ptr<V>(rej), thrust::device_ptr<V>(rej + (n - c)), first + c);
  return first + c;
}
template <class It> struct unwraps_to_pointer : std::is_pointer<typename thrust::detail::unwrap_iterator<It>::type> {};
}  // namespace detail
template <class D, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category,
          typename std::enable_if<!(detail::unwraps_to_pointer<It>::value && detail::unwraps_to_pointer<St>::value), int>::type = 0>
It stable_partition(const system::cdna4::execution_policy<D>& exec, It first, It last, St stencil, Pred pred) {
  return detail::stable_partition_gathered<false>(exec.derived(), first, last, stencil, pred);
}
template <class D, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category,
          typename std::enable_if<detail::unwraps_to_pointer<It>::value && detail::unwraps_to_pointer<St>::value, int>::type = 0>
It stable_partition(const system::cdna4::execution_policy<D>& exec, It first, It last, St stencil, Pred pred) {
  namespace sd = system::cdna4::detail;
  typedef typename thrust::detail::value_of<It>::type V;
  typedef typename thrust::detail::value_of<St>::type S;
  const std::int64_t n = (std::int64_t)(last - first);
  if (n <= 0) return first;
  void* s = sd::stream_of(exec.derived());
  V* data = (V*)thrust::detail::unwrap(first);
  sd::scratch_copy<V> in(data, n, s);
  sd::temporary_storage rejected((std::size_t)n * sizeof(V), s);
  const S* st = (const void*)thrust::detail::unwrap(stencil) == (const void*)data ? (const S*)in.data() : (const S*)thrust::detail::unwrap(stencil);
  const std::int64_t c = sd::partition_copy_n(exec.derived(), in.data(), st, data, static_cast<V*>(rejected.data()), n, pred);
  if (c < n) {
    sd::throw_on_error(thrust_cdna4_memcpy_dtod(data + c, rejected.data(), (std::size_t)(n - c) * sizeof(V), s), "partition: append");
    sd::throw_on_error(thrust_cdna4_stream_synchronize(s), "partition: failed to synchronize");
  }
  return first + c;
}
template <class D, class It, class Pred, typename std::enable_if<detail::unwraps_to_pointer<It>::value, int>::type = 0>
It stable_partition(const system::cdna4::execution_policy<D>& exec, It first, It last, Pred pred) {
  return stable_partition(exec, first, last, first, pred);
}
template <class D, class It, class Pred, typename std::enable_if<!detail::unwraps_to_pointer<It>::value, int>::type = 0>
It stable_partition(const system::cdna4::execution_policy<D>& exec, It first, It last, Pred pred) {
  return detail::stable_partition_gathered<true>(exec.derived(), first, last, first, pred);
}
}}  // namespace system::cdna4
}  // namespace thrust
