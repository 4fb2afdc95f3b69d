// thrust::cdna4::histogram_even — extension of the cdna4 system (the reference has no
// histogram algorithm; its example builds one from sort + upper_bound + adjacent_difference,
// examples/histogram.cu:60-101).  counts[b] = number of samples x with
// floor((x - lower) * num_bins / (upper - lower)) == b; samples outside [lower, upper) are dropped.
#pragma once
#include <cstdint>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>

namespace thrust { namespace cdna4 {

template <class D, class It, class CountIt>
void histogram_even(const thrust::system::cdna4::execution_policy<D>& exec, It first, It last, CountIt counts,
                    int num_bins, double lower, double upper) {
  typedef typename std::remove_const<typename thrust::detail::value_of<It>::type>::type T;
  namespace d = thrust::system::cdna4::detail;
  static_assert(d::dtype_of<T>::supported, "cdna4 histogram_even: samples must be an arithmetic type");
  static_assert(sizeof(typename thrust::detail::value_of<CountIt>::type) == 4, "cdna4 histogram_even: 32-bit counters");
  void* s = d::stream_of(exec.derived());
  std::size_t bytes = 0;
  d::throw_on_error(thrust_cdna4_histogram_even(nullptr, &bytes, d::dtype_of<T>::value, thrust::detail::unwrap(first),
                                                (std::int64_t)(last - first), nullptr, num_bins, lower, upper, s),
                    "histogram_even: temporary storage query");
  d::temporary_storage tmp(bytes, exec.derived());
  d::throw_on_error(thrust_cdna4_histogram_even(tmp.data(), &bytes, d::dtype_of<T>::value, thrust::detail::unwrap(first),
                                                (std::int64_t)(last - first),
                                                reinterpret_cast<std::uint32_t*>(thrust::detail::unwrap(counts)), num_bins,
                                                lower, upper, s), "histogram_even: launch");
  d::synchronize_optional(exec.derived(), "histogram_even: failed to synchronize");
}
template <class It, class CountIt>
void histogram_even(It first, It last, CountIt counts, int num_bins, double lower, double upper) {
  histogram_even(thrust::device, first, last, counts, num_bins, lower, upper);
}

}}  // namespace thrust::cdna4
