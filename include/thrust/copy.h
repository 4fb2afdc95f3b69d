// thrust::copy between and within systems for contiguous ranges of arithmetic elements
// (thrust/copy.h; thrust/system/cuda/detail/internal/copy_cross_system.h:89-223).
#pragma once
#include <algorithm>
#include <iterator>
#include <memory>
#include <vector>
#include <thrust/device_ptr.h>

namespace thrust {
namespace system { namespace cdna4 { namespace detail {
inline void copy_bytes(void* dst, const void* src, std::size_t bytes, int kind) {
  if (!bytes) return;
  int rc = kind == 0   ? thrust_cdna4_memcpy_htod(dst, src, bytes, nullptr)
           : kind == 1 ? thrust_cdna4_memcpy_dtoh(dst, src, bytes, nullptr)
                       : thrust_cdna4_memcpy_dtod(dst, src, bytes, nullptr);
  throw_on_error(rc, "copy");
  throw_on_error(thrust_cdna4_stream_synchronize(nullptr), "copy");
}
}}}  // namespace system::cdna4::detail

// device -> device
namespace detail {
template <class T, class U>
device_ptr<U> copy_device_range(device_ptr<T> first, device_ptr<T> last, device_ptr<U> out, std::true_type) {
  system::cdna4::detail::copy_bytes(out.get(), first.get(), (last - first) * sizeof(U), 2);
  return out + (last - first);
}
// another element type: converted element by element on the device (defined below, once the device
// system's copy is declared)
template <class T, class U>
device_ptr<U> copy_device_range(device_ptr<T> first, device_ptr<T> last, device_ptr<U> out, std::false_type);
}  // namespace detail
template <class T, class U>
device_ptr<U> copy(device_ptr<T> first, device_ptr<T> last, device_ptr<U> out) {
  return detail::copy_device_range(first, last, out, std::is_same<typename std::remove_const<T>::type, U>());
}
// device -> host (contiguous host output: raw pointer or vector iterator)
template <class T, class OutIt, class = typename std::enable_if<!system::cdna4::detail::is_device_iterator<OutIt>::value>::type>
OutIt copy(device_ptr<T> first, device_ptr<T> last, OutIt out) {
  typedef typename std::remove_const<T>::type V;
  const std::size_t n = (std::size_t)(last - first);
  std::unique_ptr<V[]> tmp(new V[n]);
  system::cdna4::detail::copy_bytes(tmp.get(), first.get(), n * sizeof(V), 1);
  return std::copy(tmp.get(), tmp.get() + n, out);
}
// host -> device
template <class InIt, class U, class = typename std::enable_if<!system::cdna4::detail::is_device_iterator<InIt>::value>::type>
device_ptr<U> copy(InIt first, InIt last, device_ptr<U> out) {
  const std::size_t n = (std::size_t)std::distance(first, last);
  std::unique_ptr<U[]> tmp(new U[n]);  // (not std::vector: its bool specialisation is no array)
  std::copy(first, last, tmp.get());
  system::cdna4::detail::copy_bytes(out.get(), tmp.get(), n * sizeof(U), 0);
  return out + n;
}
// host -> host
template <class InIt, class OutIt,
          class = typename std::enable_if<(!system::cdna4::detail::is_device_iterator<InIt>::value ||
                                           system::cdna4::detail::is_any_system_iterator<InIt>::value) &&
                                          !system::cdna4::detail::is_device_iterator<OutIt>::value>::type>
OutIt copy(InIt first, InIt last, OutIt out) {
  return std::copy(first, last, out);
}
}  // namespace thrust

// thrust::copy_if, with and without a stencil (thrust/copy.h; thrust/system/cuda/detail/copy_if.h):
// stable compaction with a user predicate — kernel templates on device ranges.
#include <thrust/execution_policy.h>
#include <thrust/detail/iterator_util.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>
#include <thrust/system/cdna4/detail/copy_if.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/copy.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class Pred>
Out copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out out, Pred pred) {
  return copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, out, pred);
}
template <class D, class In, class St, class Out, class Pred>
Out copy_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out out, Pred pred) {
  return copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, out, pred);
}
template <class In, class Out, class Pred>
Out copy_if(const system::cpp::detail::par_t&, In first, In last, Out out, Pred pred) { return std::copy_if(first, last, out, pred); }
template <class In, class St, class Out, class Pred>
Out copy_if(const system::cpp::detail::par_t&, In first, In last, St stencil, Out out, Pred pred) {
  for (; first != last; ++first, ++stencil) if (pred(*stencil)) { *out = *first; ++out; }
  return out;
}
template <class In, class Out, class Pred, detail::enable_if_device<In, Out, Pred> = 0> Out copy_if(In f, In l, Out o, Pred p) { return copy_if(typename detail::implicit_policy<In, Out, Pred>::type(), f, l, o, p); }
template <class In, class Out, class Pred, detail::enable_if_host<In, Out, Pred> = 0> Out copy_if(In f, In l, Out o, Pred p) { return copy_if(host, f, l, o, p); }
template <class In, class St, class Out, class Pred, detail::enable_if_device<In, St, Out, Pred> = 0,
          class = typename std::iterator_traits<St>::iterator_category>
Out copy_if(In f, In l, St s, Out o, Pred p) { return copy_if(typename detail::implicit_policy<In, St, Out, Pred>::type(), f, l, s, o, p); }
template <class In, class St, class Out, class Pred, detail::enable_if_host<In, St, Out, Pred> = 0,
          class = typename std::iterator_traits<St>::iterator_category>
Out copy_if(In f, In l, St s, Out o, Pred p) { return copy_if(host, f, l, s, o, p); }

// thrust::copy from a fancy device iterator (counting, transform, zip, permutation ...): an
// identity transform on the device; a host destination receives it through a device temporary.
namespace detail {
template <class It> struct is_fancy_device_iterator { static constexpr bool value = system::cdna4::detail::is_device_iterator<It>::value; };
template <class T> struct is_fancy_device_iterator<device_ptr<T>> { static constexpr bool value = false; };
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/copy.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/copy.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out>
Out copy(const detail::execution_policy_base<D>& exec, In first, In last, Out out) {
  return copy(detail::derived_cast(detail::strip_const(exec)), first, last, out);
}
template <class D, class T>
device_ptr<typename std::remove_const<T>::type> copy(const detail::execution_policy_base<D>& exec, device_ptr<T> first, device_ptr<T> last, device_ptr<typename std::remove_const<T>::type> out) {
  return copy(detail::derived_cast(detail::strip_const(exec)), first, last, out);
}

template <class In, class Out>
Out copy(const system::cpp::detail::par_t&, In first, In last, Out out) { return std::copy(first, last, out); }
template <class In, class Out,
          typename std::enable_if<detail::is_fancy_device_iterator<In>::value && system::cdna4::detail::is_device_iterator<Out>::value, int>::type = 0>
Out copy(In first, In last, Out out) { return copy(typename detail::implicit_policy<In>::type(), first, last, out); }
template <class In, class Out,
          typename std::enable_if<detail::is_fancy_device_iterator<In>::value && !system::cdna4::detail::is_any_system_iterator<In>::value &&
                                      !system::cdna4::detail::is_device_iterator<Out>::value, long>::type = 0>
Out copy(In first, In last, Out out) {
  typedef typename detail::value_of<In>::type V;
  const std::size_t n = (std::size_t)(last - first);
  system::cdna4::detail::temporary_storage staging(n * sizeof(V), static_cast<void*>(nullptr));
  V* tmp = static_cast<V*>(staging.data());
  copy(device, first, last, device_ptr<V>(tmp));
  std::unique_ptr<V[]> host(new V[n]);
  system::cdna4::detail::copy_bytes(host.get(), tmp, n * sizeof(V), 1);
  return std::copy(host.get(), host.get() + n, out);
}
namespace detail {
template <class T, class U>
device_ptr<U> copy_device_range(device_ptr<T> first, device_ptr<T> last, device_ptr<U> out, std::false_type) {
  return copy(device, first, last, out);
}
}  // namespace detail
// The remaining pairs of systems without a policy.  A contiguous device range into a device output
// that is no plain pointer (a zip or transform-output iterator over device memory, a discard
// iterator): the device system's copy.
template <class T, class Out,
          typename std::enable_if<system::cdna4::detail::is_device_iterator<Out>::value, char>::type = 0>
Out copy(device_ptr<T> first, device_ptr<T> last, Out out) { return copy(typename detail::implicit_policy<device_ptr<T>, Out>::type(), first, last, out); }
// A host range (or a counting / constant range) into such an output: a discard iterator drops it on
// the host; otherwise the elements are staged in device memory and copied there.
template <class In, class Out,
          typename std::enable_if<(!system::cdna4::detail::is_device_iterator<In>::value) &&
                                      system::cdna4::detail::is_device_iterator<Out>::value, short>::type = 0>
Out copy(In first, In last, Out out) {
  typedef typename detail::value_of<In>::type V;
  const std::size_t n = (std::size_t)std::distance(first, last);
  if (system::cdna4::detail::is_any_system_iterator<Out>::value || n == 0) return out + n;
  std::unique_ptr<V[]> host(new V[n]);
  std::copy(first, last, host.get());
  system::cdna4::detail::temporary_storage staging(n * sizeof(V), static_cast<void*>(nullptr));
  V* tmp = static_cast<V*>(staging.data());
  system::cdna4::detail::copy_bytes(tmp, host.get(), n * sizeof(V), 0);
  Out end = copy(device, device_ptr<V>(tmp), device_ptr<V>(tmp + n), out);
  system::cdna4::detail::throw_on_error(thrust_cdna4_stream_synchronize(nullptr), "copy");
  return end;
}
namespace detail {
// first + n, also for iterators that only step (a std::list's)
template <class It, class N> inline auto plus_n(It it, N n, int) -> decltype(It(it + n)) { return it + n; }
template <class It, class N> inline It plus_n(It it, N n, long) { std::advance(it, n); return it; }
}  // namespace detail
namespace detail {
template <class Policy, class In, class Size, class Out>
Out composed_copy_n(const Policy& exec, In first, Size n, Out out) { return thrust::copy(exec, first, detail::plus_n(first, n, 0), out); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Size, class Out>
Out copy_n(execution_policy<D_>& exec, In first, Size n, Out out) { return thrust::detail::composed_copy_n(exec, first, n, out); }
}}  // namespace system::cdna4
template <class D_, class In, class Size, class Out>
Out copy_n(const detail::execution_policy_base<D_>& exec, In first, Size n, Out out) { return copy_n(detail::derived_cast(detail::strip_const(exec)), first, n, out); }
template <class In, class Size, class Out>
Out copy_n(const system::cpp::detail::par_t& exec, In first, Size n, Out out) { return detail::composed_copy_n(exec, first, n, out); }
namespace detail {
// iterators retagged with a user's policy type select that policy (testing/copy_n.cu:268-285)
template <class... Its> struct has_user_policy {
  static constexpr bool value = !std::is_same<typename implicit_policy<Its...>::type, system::cdna4::detail::par_t>::value;
};
}  // namespace detail
template <class In, class Size, class Out, typename std::enable_if<!detail::is_policy<In>::value && !detail::has_user_policy<In, Out>::value, int>::type = 0>
Out copy_n(In first, Size n, Out out) { return thrust::copy(first, detail::plus_n(first, n, 0), out); }
template <class In, class Size, class Out, typename std::enable_if<!detail::is_policy<In>::value && detail::has_user_policy<In, Out>::value, int>::type = 0>
Out copy_n(In first, Size n, Out out) { return copy_n(typename detail::implicit_policy<In, Out>::type(), first, n, out); }
}  // namespace thrust
