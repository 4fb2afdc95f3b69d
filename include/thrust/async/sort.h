// thrust::async::sort / stable_sort (thrust/async/sort.h; thrust/system/cuda/detail/async/sort.h).
#pragma once
#include <thrust/event.h>
#include <thrust/sort.h>

namespace thrust { namespace async {
template <class Policy, class It, class Compare, thrust::detail::enable_if_policy<Policy> = 0>
device_event stable_sort(const Policy& exec, It first, It last, Compare comp) {
  auto signal = system::cdna4::detail::make_signal(exec);
  thrust::stable_sort(thrust::cdna4::par_nosync.on(signal->stream()), first, last, comp);
  return device_event(std::move(signal));
}
template <class Policy, class It, thrust::detail::enable_if_policy<Policy> = 0>
device_event stable_sort(const Policy& exec, It first, It last) {
  return async::stable_sort(exec, first, last, thrust::less<typename thrust::detail::value_of<It>::type>());
}
template <class It, class Compare, thrust::detail::enable_if_device<It> = 0>
device_event stable_sort(It first, It last, Compare comp) { return async::stable_sort(thrust::device, first, last, comp); }
template <class It>
device_event stable_sort(It first, It last) { return async::stable_sort(thrust::device, first, last); }

template <class Policy, class It, class Compare, thrust::detail::enable_if_policy<Policy> = 0>
device_event sort(const Policy& exec, It first, It last, Compare comp) { return async::stable_sort(exec, first, last, comp); }
template <class Policy, class It, thrust::detail::enable_if_policy<Policy> = 0>
device_event sort(const Policy& exec, It first, It last) { return async::stable_sort(exec, first, last); }
template <class It, class Compare, thrust::detail::enable_if_device<It> = 0>
device_event sort(It first, It last, Compare comp) { return async::stable_sort(thrust::device, first, last, comp); }
template <class It>
device_event sort(It first, It last) { return async::stable_sort(thrust::device, first, last); }
}}  // namespace thrust::async
