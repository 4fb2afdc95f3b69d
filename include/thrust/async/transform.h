// thrust::async::transform (thrust/async/transform.h).
#pragma once
#include <thrust/event.h>
#include <thrust/transform.h>

namespace thrust { namespace async {
template <class Policy, class In, class Out, class F, thrust::detail::enable_if_policy<Policy> = 0>
device_event transform(const Policy& exec, In first, In last, Out out, F f) {
  auto signal = system::cdna4::detail::make_signal(exec);
  thrust::transform(thrust::cdna4::par_nosync.on(signal->stream()), first, last, out, f);
  return device_event(std::move(signal));
}
template <class In, class Out, class F>
device_event transform(In first, In last, Out out, F f) { return async::transform(thrust::device, first, last, out, f); }
}}  // namespace thrust::async
