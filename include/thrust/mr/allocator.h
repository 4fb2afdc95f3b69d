// thrust::mr::allocator / stateless_resource_allocator (thrust/mr/allocator.h:47-260): the
// allocator face of a memory resource, for containers and for thrust::cdna4::par(alloc).
#pragma once
#include <cstddef>
#include <thrust/device_ptr.h>
#include <thrust/mr/memory_resource.h>
#include <thrust/mr/polymorphic_adaptor.h>

namespace thrust { namespace mr {
namespace detail {
template <class Pointer, class T> struct rebind_pointer;
template <class U, class T> struct rebind_pointer<U*, T> {
  typedef T* type;
  static type from_void(void* p) { return static_cast<T*>(p); }
  static void* to_void(T* p) { return const_cast<typename std::remove_const<T>::type*>(p); }
};
template <class U, class T> struct rebind_pointer<thrust::device_ptr<U>, T> {
  typedef thrust::device_ptr<T> type;
  static type from_void(thrust::device_ptr<void> p) { return type(static_cast<T*>(p.get())); }
  static thrust::device_ptr<void> to_void(type p) { return thrust::device_ptr<void>((void*)p.get()); }
};
}  // namespace detail

template <class T, class MR>
class allocator {
 public:
  typedef T value_type;
  typedef typename detail::rebind_pointer<typename MR::pointer, T>::type pointer;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  template <class U> struct rebind { typedef allocator<U, MR> other; };

  explicit allocator(MR* resource) : resource_(resource) {}
  template <class U> allocator(const allocator<U, MR>& other) : resource_(other.resource()) {}
  pointer allocate(size_type n) {
    return detail::rebind_pointer<typename MR::pointer, T>::from_void(resource_->allocate(n * sizeof(T), alignof(T)));
  }
  void deallocate(pointer p, size_type n) {
    resource_->deallocate(detail::rebind_pointer<typename MR::pointer, T>::to_void(p), n * sizeof(T), alignof(T));
  }
  size_type max_size() const { return size_type(-1) / sizeof(T); }
  MR* resource() const { return resource_; }
 private:
  MR* resource_;
};
template <class T, class U, class MR>
bool operator==(const allocator<T, MR>& a, const allocator<U, MR>& b) { return *a.resource() == *b.resource(); }
template <class T, class U, class MR>
bool operator!=(const allocator<T, MR>& a, const allocator<U, MR>& b) { return !(a == b); }

// default-constructible: uses the global instance of its resource type
template <class T, class Upstream>
class stateless_resource_allocator : public allocator<T, Upstream> {
 public:
  template <class U> struct rebind { typedef stateless_resource_allocator<U, Upstream> other; };
  stateless_resource_allocator() : allocator<T, Upstream>(get_global_resource<Upstream>()) {}
  template <class U> stateless_resource_allocator(const stateless_resource_allocator<U, Upstream>& o) : allocator<T, Upstream>(o) {}
};
// an allocator over a resource chosen at run time (thrust/mr/allocator.h:229-260)
template <class T, class Pointer>
class polymorphic_allocator : public allocator<T, polymorphic_adaptor_resource<Pointer>> {
  typedef allocator<T, polymorphic_adaptor_resource<Pointer>> base;
 public:
  template <class U> struct rebind { typedef polymorphic_allocator<U, Pointer> other; };
  polymorphic_allocator(polymorphic_adaptor_resource<Pointer>* resource) : base(resource) {}
  template <class U> polymorphic_allocator(const polymorphic_allocator<U, Pointer>& o) : base(o) {}
};
}}  // namespace thrust::mr
