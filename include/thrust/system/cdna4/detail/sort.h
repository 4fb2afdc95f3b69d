// The cdna4 device system's sort (the counterpart of thrust/system/cuda/detail/sort.h): free functions
// in the policy's namespace, found by the unqualified calls of the entry points in <thrust/sort.h>,
// which includes this file where the helpers it uses have been declared.
#pragma once
#include <thrust/sort.h>
namespace thrust {
namespace system { namespace cdna4 {
// the device system's implementations, found through the policy's type
template <class D, class It, class Compare>
void stable_sort(const system::cdna4::execution_policy<D>& exec, It first, It last, Compare comp) {
  thrust::detail::sort_range(exec.derived(), first, last, comp, typename thrust::detail::is_contiguous_device<It>::type());
}
template <class D, class It>
void stable_sort(const system::cdna4::execution_policy<D>& exec, It first, It last) {
  stable_sort(exec, first, last, less<typename thrust::detail::value_of<It>::type>());
}
// sort forwards to stable_sort, as the generic layer does (thrust/system/detail/generic/sort.inl:56-62)
template <class D, class It, class Compare>
void sort(const system::cdna4::execution_policy<D>& exec, It first, It last, Compare comp) {
  thrust::stable_sort(thrust::detail::derived_cast(thrust::detail::strip_const(exec)), first, last, comp);
}
template <class D, class It>
void sort(const system::cdna4::execution_policy<D>& exec, It first, It last) {
  thrust::stable_sort(thrust::detail::derived_cast(thrust::detail::strip_const(exec)), first, last);
}

template <class D, class KIt, class VIt, class Compare>
void stable_sort_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  thrust::detail::sort_pairs_range(exec.derived(), kfirst, klast, vfirst, comp,
                           std::integral_constant<bool, thrust::detail::is_contiguous_device<KIt>::value && thrust::detail::is_contiguous_device<VIt>::value>());
}
template <class D, class KIt, class VIt>
void stable_sort_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst) {
  stable_sort_by_key(exec, kfirst, klast, vfirst, less<typename thrust::detail::value_of<KIt>::type>());
}
template <class D, class KIt, class VIt, class Compare>
void sort_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst, Compare comp) {
  thrust::stable_sort_by_key(thrust::detail::derived_cast(thrust::detail::strip_const(exec)), kfirst, klast, vfirst, comp);
}
template <class D, class KIt, class VIt>
void sort_by_key(const system::cdna4::execution_policy<D>& exec, KIt kfirst, KIt klast, VIt vfirst) {
  thrust::stable_sort_by_key(thrust::detail::derived_cast(thrust::detail::strip_const(exec)), kfirst, klast, vfirst);
}
}}  // namespace system::cdna4
}  // namespace thrust
