// thrust::async::for_each (thrust/async/for_each.h): submits the work to a stream of its own
// and returns the event that owns it.
#pragma once
#include <thrust/event.h>
#include <thrust/for_each.h>

namespace thrust { namespace async {
template <class Policy, class It, class F, thrust::detail::enable_if_policy<Policy> = 0>
device_event for_each(const Policy& exec, It first, It last, F f) {
  auto signal = system::cdna4::detail::make_signal(exec);
  thrust::for_each(thrust::cdna4::par_nosync.on(signal->stream()), first, last, f);
  return device_event(std::move(signal));
}
template <class It, class F>
device_event for_each(It first, It last, F f) { return async::for_each(thrust::device, first, last, f); }
}}  // namespace thrust::async
