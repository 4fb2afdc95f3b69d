// thrust::universal_vector (thrust/universal_vector.h): a device_vector whose storage host code
// can address too (managed memory).  The algorithms treat it as a device range;
// raw_pointer_cast(v.data()) may be read and written on the host once device work on it is done.
// It is a class template of its own, so overloads may tell it from a device_vector.
#pragma once
#include <initializer_list>
#include <utility>
#include <thrust/device_vector.h>
#include <thrust/universal_allocator.h>
namespace thrust {
template <class T, class Alloc = universal_allocator<T>>
class universal_vector : public device_vector<T, Alloc> {
  typedef device_vector<T, Alloc> base;

 public:
  using base::base;
  universal_vector() = default;
  universal_vector(const universal_vector&) = default;
  universal_vector(universal_vector&&) = default;
  universal_vector(const base& v) : base(v) {}
  universal_vector(base&& v) : base(std::move(v)) {}
  universal_vector(std::initializer_list<T> il) : base(il) {}
  universal_vector& operator=(const universal_vector&) = default;
  universal_vector& operator=(universal_vector&&) = default;
  template <class V> universal_vector& operator=(const V& v) { base::operator=(v); return *this; }
  universal_vector& operator=(std::initializer_list<T> il) { base::operator=(base(il)); return *this; }
};
}  // namespace thrust
