// thrust::host_vector (thrust/host_vector.h): a std::vector in host memory.
#pragma once
#include <vector>
namespace thrust {
template <class T> class device_allocator;
template <class T> class device_ptr;
template <class T, class Alloc = device_allocator<T>> class device_vector;
template <class T, class Alloc = std::allocator<T>>
class host_vector : public std::vector<T, Alloc> {
  typedef std::vector<T, Alloc> base;

 public:
  using base::base;
  host_vector() = default;
  host_vector(const base& v) : base(v) {}
  template <class DA> host_vector(const device_vector<T, DA>& d);
  template <class DA> host_vector& operator=(const device_vector<T, DA>& d);
  // a contiguous device range: one copy, not an element at a time
  template <class U> host_vector(device_ptr<U> first, device_ptr<U> last);
  template <class U> void assign(device_ptr<U> first, device_ptr<U> last) { host_vector tmp(first, last); this->swap(tmp); }
  using base::assign;
};
}  // namespace thrust
#include <thrust/detail/vector_common.h>
