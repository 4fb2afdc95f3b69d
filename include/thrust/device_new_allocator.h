// thrust::device_new_allocator (thrust/device_new_allocator.h): an allocator over
// thrust::device_new / device_delete (storage comes back value-initialised).
#pragma once
#include <cstddef>
#include <limits>
#include <thrust/device_delete.h>
#include <thrust/device_new.h>
#include <thrust/device_ptr.h>
namespace thrust {
template <class T>
class device_new_allocator {
 public:
  typedef T value_type;
  typedef device_ptr<T> pointer;
  typedef device_ptr<const T> const_pointer;
  typedef device_reference<T> reference;
  typedef device_reference<const T> const_reference;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  template <class U> struct rebind { typedef device_new_allocator<U> other; };
  device_new_allocator() {}
  device_new_allocator(const device_new_allocator&) {}
  template <class U> device_new_allocator(const device_new_allocator<U>&) {}
  pointer allocate(size_type n, const void* = nullptr) {
    if (n > max_size()) throw std::bad_alloc();
    return device_new<T>(n);
  }
  void deallocate(pointer p, size_type n) { device_delete(p, n); }
  size_type max_size() const { return std::numeric_limits<size_type>::max() / sizeof(T); }
  bool operator==(const device_new_allocator&) const { return true; }
  bool operator!=(const device_new_allocator&) const { return false; }
};
}  // namespace thrust
