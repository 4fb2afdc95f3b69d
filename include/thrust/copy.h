// thrust::copy between and within systems for contiguous ranges of arithmetic elements
// (thrust/copy.h; thrust/system/cuda/detail/internal/copy_cross_system.h:89-223).
#pragma once
#include <algorithm>
#include <iterator>
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
template <class T, class U>
device_ptr<U> copy(device_ptr<T> first, device_ptr<T> last, device_ptr<U> out) {
  static_assert(std::is_same<typename std::remove_const<T>::type, U>::value, "element types must match");
  system::cdna4::detail::copy_bytes(out.get(), first.get(), (last - first) * sizeof(U), 2);
  return out + (last - first);
}
// device -> host (contiguous host output: raw pointer or vector iterator)
template <class T, class OutIt, class = typename std::enable_if<!system::cdna4::detail::is_device_iterator<OutIt>::value>::type>
OutIt copy(device_ptr<T> first, device_ptr<T> last, OutIt out) {
  typedef typename std::remove_const<T>::type V;
  std::vector<V> tmp(last - first);
  system::cdna4::detail::copy_bytes(tmp.data(), first.get(), tmp.size() * sizeof(V), 1);
  return std::copy(tmp.begin(), tmp.end(), out);
}
// host -> device
template <class InIt, class U, class = typename std::enable_if<!system::cdna4::detail::is_device_iterator<InIt>::value>::type>
device_ptr<U> copy(InIt first, InIt last, device_ptr<U> out) {
  std::vector<U> tmp(first, last);
  system::cdna4::detail::copy_bytes(out.get(), tmp.data(), tmp.size() * sizeof(U), 0);
  return out + tmp.size();
}
// host -> host
template <class InIt, class OutIt,
          class = typename std::enable_if<!system::cdna4::detail::is_device_iterator<InIt>::value &&
                                          !system::cdna4::detail::is_device_iterator<OutIt>::value>::type>
OutIt copy(InIt first, InIt last, OutIt out) {
  return std::copy(first, last, out);
}
}  // namespace thrust
