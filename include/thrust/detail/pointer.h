// thrust::pointer<Element, Tag, Reference, Derived> (thrust/memory.h:77-170,
// thrust/detail/pointer.h:36-250): a pointer that carries the system of the memory it points to in
// its type.  Tag is a system tag or a user's policy type; with the host system's tag the pointer
// dereferences to a plain reference, otherwise to a thrust::device_reference (one element copied
// per access on the host, the element itself in a kernel).  User pointer classes derive from it and
// name themselves as Derived, so that arithmetic on them returns their own type.
#pragma once
#include <cstddef>
#include <iterator>
#include <type_traits>
#include <thrust/detail/iterator_util.h>
#include <thrust/device_ptr.h>
#include <thrust/iterator/detail/fancy_base.h>
namespace thrust {
template <class Element, class Tag, class Reference = use_default, class Derived = use_default>
class pointer;
namespace detail {
template <class Tag> struct is_host_tag : std::is_base_of<system::cpp::tag, Tag> {};
template <class Element, class Tag, class Reference> struct pointer_reference {
  typedef typename std::conditional<is_host_tag<Tag>::value, typename std::add_lvalue_reference<Element>::type,
                                    thrust::device_reference<Element>>::type deduced;
  typedef typename std::conditional<std::is_same<Reference, use_default>::value, deduced, Reference>::type type;
};
template <class Tag, class Reference> struct pointer_reference<void, Tag, Reference> { typedef void type; };
template <class Tag, class Reference> struct pointer_reference<const void, Tag, Reference> { typedef void type; };
template <class R, class E> struct make_pointer_reference { THRUST_CDNA4_HD static R from(E* p) { return R(p); } };
template <class E> struct make_pointer_reference<E&, E> { THRUST_CDNA4_HD static E& from(E* p) { return *p; } };
}  // namespace detail

template <class Element, class Tag, class Reference, class Derived>
class pointer {
  typedef typename std::conditional<std::is_same<Derived, use_default>::value, pointer, Derived>::type derived_type;
  THRUST_CDNA4_HD derived_type& self() { return static_cast<derived_type&>(*this); }
  THRUST_CDNA4_HD const derived_type& self() const { return static_cast<const derived_type&>(*this); }
  THRUST_CDNA4_HD static derived_type make(Element* p) { derived_type d; static_cast<pointer&>(d).p_ = p; return d; }

 public:
  typedef Element element_type;
  typedef typename std::remove_cv<Element>::type value_type;
  typedef typename detail::pointer_reference<Element, Tag, Reference>::type reference;
  typedef Element* raw_pointer;
  typedef std::ptrdiff_t difference_type;
  typedef derived_type pointer_type;
  typedef std::random_access_iterator_tag iterator_category;
  typedef Tag system_tag;
  typedef std::integral_constant<bool, !detail::is_host_tag<Tag>::value> thrust_system_is_device;

  THRUST_CDNA4_HD pointer() : p_(nullptr) {}
  THRUST_CDNA4_HD pointer(std::nullptr_t) : p_(nullptr) {}
  template <class Other, class = typename std::enable_if<std::is_convertible<Other*, Element*>::value>::type>
  THRUST_CDNA4_HD explicit pointer(Other* p) : p_(p) {}
  // from a pointer of another element type or tag, when the raw pointers and the tags convert
  template <class E2, class T2, class R2, class D2,
            class = typename std::enable_if<std::is_convertible<E2*, Element*>::value && std::is_convertible<T2, Tag>::value>::type>
  THRUST_CDNA4_HD pointer(const pointer<E2, T2, R2, D2>& o) : p_(o.get()) {}
  template <class E2, class T2, class R2, class D2,
            class = typename std::enable_if<std::is_convertible<E2*, Element*>::value && std::is_convertible<T2, Tag>::value>::type>
  THRUST_CDNA4_HD derived_type& operator=(const pointer<E2, T2, R2, D2>& o) { p_ = o.get(); return self(); }
  THRUST_CDNA4_HD derived_type& operator=(std::nullptr_t) { p_ = nullptr; return self(); }

  THRUST_CDNA4_HD Element* get() const { return p_; }
  THRUST_CDNA4_HD Element* operator->() const { return p_; }
  THRUST_CDNA4_HD explicit operator bool() const { return p_ != nullptr; }
  template <class E = Element>
  THRUST_CDNA4_HD typename detail::pointer_reference<E, Tag, Reference>::type operator*() const {
    return detail::make_pointer_reference<typename detail::pointer_reference<E, Tag, Reference>::type, E>::from(p_);
  }
  template <class E = Element>
  THRUST_CDNA4_HD typename detail::pointer_reference<E, Tag, Reference>::type operator[](difference_type i) const {
    return detail::make_pointer_reference<typename detail::pointer_reference<E, Tag, Reference>::type, E>::from(p_ + i);
  }
  template <class E = Element>
  THRUST_CDNA4_HD static derived_type pointer_to(typename std::enable_if<!std::is_void<E>::value, E>::type& r) { return make(&r); }

  THRUST_CDNA4_HD derived_type& operator++() { ++p_; return self(); }
  THRUST_CDNA4_HD derived_type operator++(int) { derived_type t = self(); ++p_; return t; }
  THRUST_CDNA4_HD derived_type& operator--() { --p_; return self(); }
  THRUST_CDNA4_HD derived_type operator--(int) { derived_type t = self(); --p_; return t; }
  THRUST_CDNA4_HD derived_type& operator+=(difference_type n) { p_ += n; return self(); }
  THRUST_CDNA4_HD derived_type& operator-=(difference_type n) { p_ -= n; return self(); }
  THRUST_CDNA4_HD friend derived_type operator+(const pointer& a, difference_type n) { return make(a.p_ + n); }
  THRUST_CDNA4_HD friend derived_type operator+(difference_type n, const pointer& a) { return make(a.p_ + n); }
  THRUST_CDNA4_HD friend derived_type operator-(const pointer& a, difference_type n) { return make(a.p_ - n); }
  THRUST_CDNA4_HD friend difference_type operator-(const pointer& a, const pointer& b) { return a.p_ - b.p_; }
  THRUST_CDNA4_HD friend bool operator==(const pointer& a, const pointer& b) { return a.p_ == b.p_; }
  THRUST_CDNA4_HD friend bool operator!=(const pointer& a, const pointer& b) { return a.p_ != b.p_; }
  THRUST_CDNA4_HD friend bool operator<(const pointer& a, const pointer& b) { return a.p_ < b.p_; }
  THRUST_CDNA4_HD friend bool operator>(const pointer& a, const pointer& b) { return a.p_ > b.p_; }
  THRUST_CDNA4_HD friend bool operator<=(const pointer& a, const pointer& b) { return a.p_ <= b.p_; }
  THRUST_CDNA4_HD friend bool operator>=(const pointer& a, const pointer& b) { return a.p_ >= b.p_; }
  THRUST_CDNA4_HD friend bool operator==(const pointer& a, std::nullptr_t) { return a.p_ == nullptr; }
  THRUST_CDNA4_HD friend bool operator==(std::nullptr_t, const pointer& a) { return a.p_ == nullptr; }
  THRUST_CDNA4_HD friend bool operator!=(const pointer& a, std::nullptr_t) { return a.p_ != nullptr; }
  THRUST_CDNA4_HD friend bool operator!=(std::nullptr_t, const pointer& a) { return a.p_ != nullptr; }

 private:
  Element* p_;
};
template <class E, class T, class R, class D>
THRUST_CDNA4_HD inline E* raw_pointer_cast(const pointer<E, T, R, D>& p) { return p.get(); }
template <class Ch, class Tr, class E, class T, class R, class D>
std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const pointer<E, T, R, D>& p) {
  return os << static_cast<const void*>(p.get());
}

namespace detail {
// kernels receive the raw pointer; a call without a policy runs under the pointer's tag when that
// is a policy type of the user's
template <class E, class T, class R, class D> struct unwrap_iterator<thrust::pointer<E, T, R, D>> {
  typedef E* type;
  static type apply(const thrust::pointer<E, T, R, D>& p) { return p.get(); }
};
template <class E, class T, class R, class D, class... Rest> struct implicit_policy<thrust::pointer<E, T, R, D>, Rest...> {
  typedef typename std::conditional<std::is_base_of<system::cdna4::execution_policy<T>, T>::value, T,
                                    typename implicit_policy<Rest...>::type>::type type;
};
}  // namespace detail
}  // namespace thrust
// (the class cannot have a member named `pointer`, its own name, so the standard traits are given here)
namespace std {
template <class E, class T, class R, class D>
struct iterator_traits<thrust::pointer<E, T, R, D>> {
  typedef typename thrust::pointer<E, T, R, D>::difference_type difference_type;
  typedef typename thrust::pointer<E, T, R, D>::value_type value_type;
  typedef thrust::pointer<E, T, R, D> pointer;
  typedef typename thrust::pointer<E, T, R, D>::reference reference;
  typedef std::random_access_iterator_tag iterator_category;
};
}  // namespace std
