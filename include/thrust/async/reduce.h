// thrust::async::reduce / reduce_into (thrust/async/reduce.h;
// thrust/system/cuda/detail/async/reduce.h): the sum is produced on the device in stream order;
// reduce returns a future that owns its storage, reduce_into writes to the caller's.
#pragma once
#include <thrust/event.h>
#include <thrust/reduce.h>

namespace thrust { namespace async {
template <class Policy, class It, class Out, class T, class Op, thrust::detail::enable_if_policy<Policy> = 0>
device_event reduce_into(const Policy& exec, It first, It last, Out out, T init, Op op) {
  namespace sd = system::cdna4::detail;
  THRUST_CDNA4_NEEDS_HIPCC(Op);
  auto signal = sd::make_signal(exec);
#if defined(__HIPCC__)
  typedef typename thrust::detail::unwrap_iterator<It>::type In;
  typedef typename thrust::detail::value_of<It>::type V;
  sd::generic::transform_reduce_into(signal->stream(), (std::int64_t)(last - first),
                                     sd::load_transform<In, thrust::identity<V>, T>{thrust::detail::unwrap(first), thrust::identity<V>()}, init, op,
                                     (T*)thrust::detail::unwrap(out));
#else
  (void)first; (void)last; (void)out; (void)init; (void)op;
#endif
  return device_event(std::move(signal));
}
template <class Policy, class It, class Out, class T, thrust::detail::enable_if_policy<Policy> = 0>
device_event reduce_into(const Policy& exec, It first, It last, Out out, T init) { return async::reduce_into(exec, first, last, out, init, thrust::plus<T>()); }
template <class Policy, class It, class Out, thrust::detail::enable_if_policy<Policy> = 0>
device_event reduce_into(const Policy& exec, It first, It last, Out out) {
  typedef typename thrust::detail::value_of<It>::type T;
  return async::reduce_into(exec, first, last, out, T(), thrust::plus<T>());
}
template <class It, class Out, class T, class Op, thrust::detail::enable_if_device<It> = 0>
device_event reduce_into(It first, It last, Out out, T init, Op op) { return async::reduce_into(thrust::device, first, last, out, init, op); }
template <class It, class Out, class T, thrust::detail::enable_if_device<It> = 0>
device_event reduce_into(It first, It last, Out out, T init) { return async::reduce_into(thrust::device, first, last, out, init); }
template <class It, class Out, thrust::detail::enable_if_device<It> = 0>
device_event reduce_into(It first, It last, Out out) { return async::reduce_into(thrust::device, first, last, out); }

template <class Policy, class It, class T, class Op, thrust::detail::enable_if_policy<Policy> = 0>
device_future<T> reduce(const Policy& exec, It first, It last, T init, Op op) {
  namespace sd = system::cdna4::detail;
  THRUST_CDNA4_NEEDS_HIPCC(Op);
  auto signal = sd::make_signal(exec);
  void* stream = signal->stream();
  T* result = static_cast<T*>(sd::malloc_bytes(sizeof(T), stream));
  signal->keep_alive(std::shared_ptr<void>(result, [stream](void* p) { sd::free_bytes(p, stream); }));
#if defined(__HIPCC__)
  typedef typename thrust::detail::unwrap_iterator<It>::type In;
  typedef typename thrust::detail::value_of<It>::type V;
  sd::generic::transform_reduce_into(stream, (std::int64_t)(last - first),
                                     sd::load_transform<In, thrust::identity<V>, T>{thrust::detail::unwrap(first), thrust::identity<V>()}, init, op, result);
#else
  (void)first; (void)last; (void)init; (void)op;
#endif
  return device_future<T>(std::move(signal), result);
}
template <class Policy, class It, class T, thrust::detail::enable_if_policy<Policy> = 0>
device_future<T> reduce(const Policy& exec, It first, It last, T init) { return async::reduce(exec, first, last, init, thrust::plus<T>()); }
template <class Policy, class It, thrust::detail::enable_if_policy<Policy> = 0>
device_future<typename thrust::detail::value_of<It>::type> reduce(const Policy& exec, It first, It last) {
  typedef typename thrust::detail::value_of<It>::type T;
  return async::reduce(exec, first, last, T(), thrust::plus<T>());
}
template <class It, class T, class Op, thrust::detail::enable_if_device<It> = 0>
device_future<T> reduce(It first, It last, T init, Op op) { return async::reduce(thrust::device, first, last, init, op); }
template <class It, class T, thrust::detail::enable_if_device<It> = 0>
device_future<T> reduce(It first, It last, T init) { return async::reduce(thrust::device, first, last, init); }
template <class It, thrust::detail::enable_if_device<It> = 0>
device_future<typename thrust::detail::value_of<It>::type> reduce(It first, It last) { return async::reduce(thrust::device, first, last); }
}}  // namespace thrust::async
