// thrust::fill (thrust/fill.h; thrust/system/cuda/detail/fill.h:61-75).
#pragma once
#include <algorithm>
#include <thrust/device_ptr.h>
namespace thrust {
template <class T, class V>
void fill(device_ptr<T> first, device_ptr<T> last, const V& value) {
  const T v = static_cast<T>(value);
  if (last - first <= 0) return;
  system::cdna4::detail::throw_on_error(
      thrust_cdna4_fill(first.get(), &v, (int)sizeof(T), (int64_t)(last - first), nullptr), "fill");
  system::cdna4::detail::throw_on_error(thrust_cdna4_stream_synchronize(nullptr), "fill");
}
template <class It, class V, class = typename std::enable_if<!system::cdna4::detail::is_device_iterator<It>::value>::type>
void fill(It first, It last, const V& value) { std::fill(first, last, value); }
}  // namespace thrust
