// thrust::device_delete (thrust/device_delete.h): the partner of device_new — destroys n objects
// (a no-op for the trivially destructible types device storage holds) and frees their storage.
#pragma once
#include <cstddef>
#include <type_traits>
#include <thrust/device_free.h>
#include <thrust/device_ptr.h>
namespace thrust {
template <class T>
inline void device_delete(device_ptr<T> ptr, const std::size_t n = 1) {
  static_assert(std::is_trivially_destructible<T>::value, "cdna4: objects in device memory must be trivially destructible");
  (void)n;
  device_free(ptr);
}
}  // namespace thrust
