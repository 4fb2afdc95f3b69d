// thrust::async::inclusive_scan / exclusive_scan (thrust/async/scan.h).
#pragma once
#include <thrust/event.h>
#include <thrust/scan.h>

namespace thrust { namespace async {
template <class Policy, class In, class Out, class Op, thrust::detail::enable_if_policy<Policy> = 0>
device_event inclusive_scan(const Policy& exec, In first, In last, Out out, Op op) {
  auto signal = system::cdna4::detail::make_signal(exec);
  thrust::inclusive_scan(thrust::cdna4::par_nosync.on(signal->stream()), first, last, out, op);
  return device_event(std::move(signal));
}
template <class Policy, class In, class Out, thrust::detail::enable_if_policy<Policy> = 0>
device_event inclusive_scan(const Policy& exec, In first, In last, Out out) {
  return async::inclusive_scan(exec, first, last, out, thrust::plus<typename thrust::detail::value_of<In>::type>());
}
template <class In, class Out, class Op, thrust::detail::enable_if_device<In> = 0>
device_event inclusive_scan(In first, In last, Out out, Op op) { return async::inclusive_scan(thrust::device, first, last, out, op); }
template <class In, class Out, thrust::detail::enable_if_device<In> = 0>
device_event inclusive_scan(In first, In last, Out out) { return async::inclusive_scan(thrust::device, first, last, out); }

template <class Policy, class In, class Out, class T, class Op, thrust::detail::enable_if_policy<Policy> = 0>
device_event exclusive_scan(const Policy& exec, In first, In last, Out out, T init, Op op) {
  auto signal = system::cdna4::detail::make_signal(exec);
  thrust::exclusive_scan(thrust::cdna4::par_nosync.on(signal->stream()), first, last, out, init, op);
  return device_event(std::move(signal));
}
template <class Policy, class In, class Out, class T, thrust::detail::enable_if_policy<Policy> = 0>
device_event exclusive_scan(const Policy& exec, In first, In last, Out out, T init) {
  return async::exclusive_scan(exec, first, last, out, init, thrust::plus<T>());
}
template <class In, class Out, class T, class Op, thrust::detail::enable_if_device<In> = 0>
device_event exclusive_scan(In first, In last, Out out, T init, Op op) { return async::exclusive_scan(thrust::device, first, last, out, init, op); }
template <class In, class Out, class T, thrust::detail::enable_if_device<In> = 0>
device_event exclusive_scan(In first, In last, Out out, T init) { return async::exclusive_scan(thrust::device, first, last, out, init); }
}}  // namespace thrust::async
