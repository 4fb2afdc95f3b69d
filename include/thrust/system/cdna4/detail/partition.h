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
template <class D, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
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
template <class D, class It, class Pred>
It stable_partition(const system::cdna4::execution_policy<D>& exec, It first, It last, Pred pred) {
  return stable_partition(exec, first, last, first, pred);
}
}}  // namespace system::cdna4
}  // namespace thrust
