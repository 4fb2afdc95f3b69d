// The cdna4 device system's unique (the counterpart of thrust/system/cuda/detail/unique.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/unique.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/unique.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
// ---- device
template <class D, class In, class Out, class Eq>
Out unique_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out, Eq eq) {
  typedef typename thrust::detail::value_of<In>::type V;
  return out + system::cdna4::detail::unique_copy_n(exec.derived(), thrust::detail::unwrap(first), thrust::detail::unwrap(out),
                                                    (std::int64_t)(last - first), eq);
}
template <class D, class In, class Eq>
In unique(const system::cdna4::execution_policy<D>& exec, In first, In last, Eq eq) {
  typedef typename thrust::detail::value_of<In>::type V;
  const std::int64_t n = (std::int64_t)(last - first);
  system::cdna4::detail::scratch_copy<V> tmp((const V*)thrust::detail::unwrap(first), n, system::cdna4::detail::stream_of(exec.derived()));
  return first + system::cdna4::detail::unique_copy_n(exec.derived(), tmp.data(), thrust::detail::unwrap(first), n, eq);
}
template <class D, class KIn, class VIn, class KOut, class VOut, class Eq>
pair<KOut, VOut> unique_by_key_copy(const system::cdna4::execution_policy<D>& exec, KIn kfirst, KIn klast, VIn vfirst,
                                    KOut kout, VOut vout, Eq eq) {
  typedef typename thrust::detail::value_of<KIn>::type K;
  typedef typename thrust::detail::value_of<VIn>::type V;
  const std::int64_t c = system::cdna4::detail::unique_by_key_copy_n(
      exec.derived(), thrust::detail::unwrap(kfirst), thrust::detail::unwrap(vfirst), thrust::detail::unwrap(kout),
      thrust::detail::unwrap(vout), (std::int64_t)(klast - kfirst), eq);
  return thrust::make_pair(kout + c, vout + c);
}
template <class D, class KIn, class VIn, class Eq>
pair<KIn, VIn> unique_by_key(const system::cdna4::execution_policy<D>& exec, KIn kfirst, KIn klast, VIn vfirst, Eq eq) {
  typedef typename thrust::detail::value_of<KIn>::type K;
  typedef typename thrust::detail::value_of<VIn>::type V;
  const std::int64_t n = (std::int64_t)(klast - kfirst);
  void* s = system::cdna4::detail::stream_of(exec.derived());
  system::cdna4::detail::scratch_copy<K> tk((const K*)thrust::detail::unwrap(kfirst), n, s);
  system::cdna4::detail::scratch_copy<V> tv((const V*)thrust::detail::unwrap(vfirst), n, s);
  const std::int64_t c = system::cdna4::detail::unique_by_key_copy_n(exec.derived(), tk.data(), tv.data(), thrust::detail::unwrap(kfirst),
                                                                     thrust::detail::unwrap(vfirst), n, eq);
  return thrust::make_pair(kfirst + c, vfirst + c);
}
// ---- default equality
template <class D, class In, class Out, class = typename std::iterator_traits<In>::iterator_category,
          class = typename std::iterator_traits<Out>::iterator_category>
Out unique_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out out) {
  return unique_copy(exec, first, last, out, thrust::equal_to<typename thrust::detail::value_of<In>::type>());
}
template <class D, class In, class = typename std::iterator_traits<In>::iterator_category>
In unique(const system::cdna4::execution_policy<D>& exec, In first, In last) {
  return unique(exec, first, last, thrust::equal_to<typename thrust::detail::value_of<In>::type>());
}
template <class D, class KIn, class VIn, class = typename std::iterator_traits<VIn>::iterator_category>
pair<KIn, VIn> unique_by_key(const system::cdna4::execution_policy<D>& exec, KIn kfirst, KIn klast, VIn vfirst) {
  return unique_by_key(exec, kfirst, klast, vfirst, thrust::equal_to<typename thrust::detail::value_of<KIn>::type>());
}
template <class D, class KIn, class VIn, class KOut, class VOut, class = typename std::iterator_traits<VOut>::iterator_category>
pair<KOut, VOut> unique_by_key_copy(const system::cdna4::execution_policy<D>& exec, KIn kfirst, KIn klast, VIn vfirst, KOut kout, VOut vout) {
  return unique_by_key_copy(exec, kfirst, klast, vfirst, kout, vout, thrust::equal_to<typename thrust::detail::value_of<KIn>::type>());
}
}}  // namespace system::cdna4
}  // namespace thrust
