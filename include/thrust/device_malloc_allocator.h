// thrust::device_malloc_allocator (thrust/device_malloc_allocator.h): an allocator over
// thrust::device_malloc / device_free.
#pragma once
#include <cstddef>
#include <limits>
#include <thrust/device_free.h>
#include <thrust/device_malloc.h>
#include <thrust/device_ptr.h>
#include <thrust/system_error.h>
namespace thrust {
template <class T>
class device_malloc_allocator {
 public:
  typedef T value_type;
  typedef device_ptr<T> pointer;
  typedef device_ptr<const T> const_pointer;
  typedef device_reference<T> reference;
  typedef device_reference<const T> const_reference;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  template <class U> struct rebind { typedef device_malloc_allocator<U> other; };
  device_malloc_allocator() {}
  device_malloc_allocator(const device_malloc_allocator&) {}
  template <class U> device_malloc_allocator(const device_malloc_allocator<U>&) {}
  pointer allocate(size_type n, const void* = nullptr) {
    if (n > max_size()) throw std::bad_alloc();
    return device_malloc<T>(n);
  }
  void deallocate(pointer p, size_type) { device_free(p); }
  size_type max_size() const { return std::numeric_limits<size_type>::max() / sizeof(T); }
  bool operator==(const device_malloc_allocator&) const { return true; }
  bool operator!=(const device_malloc_allocator&) const { return false; }
};
}  // namespace thrust
