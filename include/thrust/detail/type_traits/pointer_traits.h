// <thrust/detail/type_traits/pointer_traits.h>: thrust::detail::pointer_traits — element type,
// raw pointer type and the conversions between a fancy pointer and the raw one, for raw pointers
// and for pointer classes with a get() member such as thrust::device_ptr
// (thrust/detail/type_traits/pointer_traits.h:190-330).  User pointer types specialise it.
#pragma once
#include <cstddef>
#include <memory>
#include <type_traits>
#include <thrust/detail/config.h>
namespace thrust { namespace detail {
template <class Ptr> struct pointer_element { typedef typename std::pointer_traits<Ptr>::element_type type; };
template <class Ptr> struct pointer_difference { typedef typename std::pointer_traits<Ptr>::difference_type type; };
template <class Ptr, class T> struct rebind_pointer { typedef typename std::pointer_traits<Ptr>::template rebind<T> type; };
template <class Ptr>
struct pointer_traits {
  typedef Ptr pointer;
  typedef typename pointer_element<Ptr>::type element_type;
  typedef typename pointer_difference<Ptr>::type difference_type;
  typedef element_type* raw_pointer;
  typedef typename Ptr::reference reference;
  template <class U> struct rebind { typedef typename rebind_pointer<Ptr, U>::type other; };
  THRUST_HOST_DEVICE static raw_pointer get(pointer p) { return p.get(); }
  template <class R = element_type>
  THRUST_HOST_DEVICE static pointer pointer_to(typename std::enable_if<!std::is_void<R>::value, R>::type& r) { return pointer(&r); }
};
template <class T>
struct pointer_traits<T*> {
  typedef T* pointer;
  typedef T element_type;
  typedef std::ptrdiff_t difference_type;
  typedef T* raw_pointer;
  typedef typename std::add_lvalue_reference<T>::type reference;
  template <class U> struct rebind { typedef U* other; };
  THRUST_HOST_DEVICE static raw_pointer get(pointer p) { return p; }
  template <class R = T>
  THRUST_HOST_DEVICE static pointer pointer_to(typename std::enable_if<!std::is_void<R>::value, R>::type& r) { return &r; }
};
template <class Ptr> struct pointer_raw_pointer { typedef typename pointer_traits<Ptr>::raw_pointer type; };
template <class Ptr> struct is_thrust_pointer : std::integral_constant<bool, !std::is_pointer<Ptr>::value> {};
}}  // namespace thrust::detail
