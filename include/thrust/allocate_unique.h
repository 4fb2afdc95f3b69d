// thrust::allocate_unique and its relatives (thrust/allocate_unique.h): std::unique_ptr whose
// deleter returns the storage to the allocator it came from.  allocate_unique<T>(alloc, args...)
// constructs T(args...), allocate_unique_n<T>(alloc, n, value) n copies of a value; the
// uninitialized_ forms only allocate.  The object is built on the host and assigned through the
// allocator's pointer, so an allocator of device memory (whose pointer is a device_ptr) works
// as well as one of host memory.
#pragma once
#include <cstddef>
#include <memory>
#include <type_traits>
#include <utility>
#include <thrust/device_ptr.h>
namespace thrust {
namespace detail {
template <class Pointer> inline bool is_null(Pointer p) { return raw_pointer_cast(p) == nullptr; }
template <class A, class T> struct rebound_allocator {
  typedef typename std::remove_cv<typename std::remove_reference<A>::type>::type::template rebind<T>::other type;
};
}  // namespace detail

template <class T, class Allocator, bool Uninitialized = false>
struct allocator_delete final {
  typedef typename detail::rebound_allocator<Allocator, T>::type allocator_type;
  typedef typename allocator_type::pointer pointer;
  template <class UAllocator> allocator_delete(UAllocator&& other) noexcept : alloc_(std::forward<UAllocator>(other)) {}
  template <class U, class UAllocator> allocator_delete(const allocator_delete<U, UAllocator>& other) noexcept : alloc_(other.get_allocator()) {}
  void operator()(pointer p) {
    // the objects are trivially destructible: nothing to destroy, initialised or not
    if (!detail::is_null(p)) alloc_.deallocate(p, 1);
  }
  allocator_type& get_allocator() noexcept { return alloc_; }
  const allocator_type& get_allocator() const noexcept { return alloc_; }
  void swap(allocator_delete& other) noexcept { using std::swap; swap(alloc_, other.alloc_); }
 private:
  allocator_type alloc_;
};
template <class T, class Allocator> using uninitialized_allocator_delete = allocator_delete<T, Allocator, true>;

template <class T, class Allocator, bool Uninitialized = false>
struct array_allocator_delete final {
  typedef typename detail::rebound_allocator<Allocator, T>::type allocator_type;
  typedef typename allocator_type::pointer pointer;
  template <class UAllocator> array_allocator_delete(UAllocator&& other, std::size_t n) noexcept : alloc_(std::forward<UAllocator>(other)), count_(n) {}
  void operator()(pointer p) {
    if (!detail::is_null(p)) alloc_.deallocate(p, count_);
  }
  allocator_type& get_allocator() noexcept { return alloc_; }
  const allocator_type& get_allocator() const noexcept { return alloc_; }
  std::size_t count() const noexcept { return count_; }
  void swap(array_allocator_delete& other) noexcept { using std::swap; swap(alloc_, other.alloc_); swap(count_, other.count_); }
 private:
  allocator_type alloc_;
  std::size_t count_;
};
template <class T, class Allocator> using uninitialized_array_allocator_delete = array_allocator_delete<T, Allocator, true>;

template <class T, class Allocator>
std::unique_ptr<T, uninitialized_allocator_delete<T, Allocator>> uninitialized_allocate_unique(const Allocator& alloc) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  return std::unique_ptr<T, uninitialized_allocator_delete<T, Allocator>>(a.allocate(1), uninitialized_allocator_delete<T, Allocator>(a));
}
template <class T, class Allocator, class... Args>
std::unique_ptr<T, allocator_delete<T, Allocator>> allocate_unique(const Allocator& alloc, Args&&... args) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  auto p = a.allocate(1);
  try {
    *p = T(std::forward<Args>(args)...);
  } catch (...) {
    a.deallocate(p, 1);
    throw;
  }
  return std::unique_ptr<T, allocator_delete<T, Allocator>>(p, allocator_delete<T, Allocator>(a));
}
template <class T, class Allocator, class Size>
std::unique_ptr<T[], uninitialized_array_allocator_delete<T, Allocator>> uninitialized_allocate_unique_n(const Allocator& alloc, Size n) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  return std::unique_ptr<T[], uninitialized_array_allocator_delete<T, Allocator>>(a.allocate(n), uninitialized_array_allocator_delete<T, Allocator>(a, n));
}
template <class T, class Allocator, class Size, class... Args>
std::unique_ptr<T[], array_allocator_delete<T, Allocator>> allocate_unique_n(const Allocator& alloc, Size n, Args&&... args) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  auto p = a.allocate(n);
  try {
    const T value(std::forward<Args>(args)...);
    for (Size i = 0; i < n; i++) p[i] = value;
  } catch (...) {
    a.deallocate(p, n);
    throw;
  }
  return std::unique_ptr<T[], array_allocator_delete<T, Allocator>>(p, array_allocator_delete<T, Allocator>(a, n));
}
}  // namespace thrust
