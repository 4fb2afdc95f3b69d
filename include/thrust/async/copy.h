// thrust::async::copy (thrust/async/copy.h; thrust/system/cuda/detail/async/copy.h): device to
// device, host to device and device to host for contiguous ranges of one trivially copyable
// type, any device iterator to a device range otherwise.  A host range must stay alive and
// untouched until the event is ready.
#pragma once
#include <algorithm>
#include <thrust/copy.h>
#include <thrust/event.h>

namespace thrust { namespace async {
namespace detail {
template <class It> struct is_device_ptr : std::false_type {};
template <class T> struct is_device_ptr<thrust::device_ptr<T>> : std::true_type {};
}  // namespace detail

// device -> device, contiguous, same type: one stream-ordered memcpy
template <class Policy, class T, thrust::detail::enable_if_policy<Policy> = 0>
device_event copy(const Policy& exec, device_ptr<T> first, device_ptr<T> last, device_ptr<typename std::remove_const<T>::type> out) {
  auto signal = system::cdna4::detail::make_signal(exec);
  system::cdna4::detail::throw_on_error(
      thrust_cdna4_memcpy_dtod(out.get(), first.get(), (std::size_t)(last - first) * sizeof(T), signal->stream()), "async copy");
  return device_event(std::move(signal));
}
// any device iterator -> device range: an identity transform
template <class Policy, class In, class Out, thrust::detail::enable_if_policy<Policy> = 0,
          typename std::enable_if<system::cdna4::detail::is_device_iterator<In>::value && system::cdna4::detail::is_device_iterator<Out>::value &&
                                  !(detail::is_device_ptr<In>::value && detail::is_device_ptr<Out>::value), int>::type = 0>
device_event copy(const Policy& exec, In first, In last, Out out) {
  auto signal = system::cdna4::detail::make_signal(exec);
  thrust::copy(thrust::cdna4::par_nosync.on(signal->stream()), first, last, out);
  return device_event(std::move(signal));
}
// host (contiguous) -> device
template <class Policy, class In, class T, thrust::detail::enable_if_policy<Policy> = 0,
          typename std::enable_if<!system::cdna4::detail::is_device_iterator<In>::value, int>::type = 0>
device_event copy(const Policy& exec, In first, In last, device_ptr<T> out) {
  static_assert(std::is_same<typename std::iterator_traits<In>::value_type, T>::value, "async copy: element types must match");
  auto signal = system::cdna4::detail::make_signal(exec);
  const std::size_t n = (std::size_t)(last - first);
  if (n)
    system::cdna4::detail::throw_on_error(thrust_cdna4_memcpy_htod(out.get(), &*first, n * sizeof(T), signal->stream()), "async copy");
  return device_event(std::move(signal));
}
// device -> host (contiguous)
template <class Policy, class T, class Out, thrust::detail::enable_if_policy<Policy> = 0,
          typename std::enable_if<!system::cdna4::detail::is_device_iterator<Out>::value, long>::type = 0>
device_event copy(const Policy& exec, device_ptr<T> first, device_ptr<T> last, Out out) {
  static_assert(std::is_same<typename std::iterator_traits<Out>::value_type, typename std::remove_const<T>::type>::value,
                "async copy: element types must match");
  auto signal = system::cdna4::detail::make_signal(exec);
  const std::size_t n = (std::size_t)(last - first);
  if (n)
    system::cdna4::detail::throw_on_error(thrust_cdna4_memcpy_dtoh(&*out, first.get(), n * sizeof(T), signal->stream()), "async copy");
  return device_event(std::move(signal));
}
// host -> host: nothing to queue; the copy is done when the event is returned
template <class Policy, class In, class Out, thrust::detail::enable_if_policy<Policy> = 0,
          typename std::enable_if<!system::cdna4::detail::is_device_iterator<In>::value &&
                                  !system::cdna4::detail::is_device_iterator<Out>::value, short>::type = 0>
device_event copy(const Policy& exec, In first, In last, Out out) {
  auto signal = system::cdna4::detail::make_signal(exec);
  signal->wait();  // what the policy depends on
  std::copy(first, last, out);
  return device_event(std::move(signal));
}
// a device iterator that is no plain pointer (counting, transform, zip ...) -> host: the general
// copy stages it; done when the event is returned
template <class Policy, class In, class Out, thrust::detail::enable_if_policy<Policy> = 0,
          typename std::enable_if<system::cdna4::detail::is_device_iterator<In>::value && !detail::is_device_ptr<In>::value &&
                                  !system::cdna4::detail::is_device_iterator<Out>::value, char>::type = 0>
device_event copy(const Policy& exec, In first, In last, Out out) {
  auto signal = system::cdna4::detail::make_signal(exec);
  signal->wait();  // what the policy depends on
  thrust::copy(first, last, out);
  return device_event(std::move(signal));
}
// a policy for the source and one for the destination (thrust/async/copy.h:96-130): the systems
// are those of the iterators, which the overloads above tell apart
namespace detail {
// of the two policies the one that carries dependencies (thrust::device.after(...)) is the one to honour
template <class From, class To>
inline const To& policy_with_dependencies(const From&, const To& to, std::false_type) { return to; }
template <class From, class To>
inline const From& policy_with_dependencies(const From& from, const To&, std::true_type) { return from; }
}  // namespace detail
template <class From, class To, class In, class Out, thrust::detail::enable_if_policy<From> = 0, thrust::detail::enable_if_policy<To> = 0>
device_event copy(const From& from, const To& to, In first, In last, Out out) {
  return async::copy(detail::policy_with_dependencies(from, to, std::is_same<From, system::cdna4::detail::execute_after>()), first, last, out);
}
template <class In, class Out,
          typename std::enable_if<!thrust::detail::is_policy<In>::value, int>::type = 0>
device_event copy(In first, In last, Out out) { return async::copy(thrust::device, first, last, out); }
}}  // namespace thrust::async
