// thrust::device_ptr / device_reference / device_pointer_cast / raw_pointer_cast
// (thrust/device_ptr.h, thrust/device_reference.h).  Reading or writing through a
// device_reference is one synchronous element copy, as in the reference
// (thrust/system/cuda/detail/get_value.h:47-58, assign_value.h).
#pragma once
#include <ostream>
#include <utility>
#include <cstddef>
#include <iterator>
#include <thrust/detail/hd.h>
#include <thrust/system/cdna4/detail/core.h>

namespace thrust {

template <class T> class device_ptr;

template <class T>
class device_reference {
 public:
  typedef typename std::remove_const<T>::type value_type;
  THRUST_CDNA4_HD explicit device_reference(T* p) : p_(p) {}
  // on the host one synchronous element copy; inside a kernel the element itself
  THRUST_CDNA4_HD operator value_type() const {
#if defined(__HIP_DEVICE_COMPILE__)
    return *p_;
#else
    value_type v;
    system::cdna4::detail::throw_on_error(thrust_cdna4_read_back(&v, p_, sizeof(T), nullptr), "get_value");
    return v;
#endif
  }
  THRUST_CDNA4_HD device_reference& operator=(const value_type& v) {
#if defined(__HIP_DEVICE_COMPILE__)
    *p_ = v;
#else
    system::cdna4::detail::throw_on_error(thrust_cdna4_memcpy_htod(p_, &v, sizeof(T), nullptr), "assign_value");
    system::cdna4::detail::throw_on_error(thrust_cdna4_stream_synchronize(nullptr), "assign_value");
#endif
    return *this;
  }
  THRUST_CDNA4_HD device_reference& operator=(const device_reference& o) { return *this = static_cast<value_type>(o); }
  // from the pointer to the element, and from a reference to an element of a convertible type
  // (thrust/device_reference.h:224-260)
  template <class P, class = decltype(static_cast<T*>(std::declval<const P&>().get()))>
  THRUST_CDNA4_HD explicit device_reference(const P& ptr) : p_(ptr.get()) {}
  template <class U, class = typename std::enable_if<std::is_convertible<U*, T*>::value && !std::is_same<U, T>::value>::type>
  THRUST_CDNA4_HD device_reference(const device_reference<U>& o) : p_((&o).get()) {}
  template <class U, class = typename std::enable_if<!std::is_same<U, T>::value>::type>
  THRUST_CDNA4_HD device_reference& operator=(const device_reference<U>& o) { return *this = static_cast<value_type>(static_cast<typename device_reference<U>::value_type>(o)); }
  THRUST_CDNA4_HD device_ptr<T> operator&() const { return device_ptr<T>(p_); }
  // read-modify-write forms (thrust/detail/reference.h:160-420)
  THRUST_CDNA4_HD device_reference& operator++() { value_type t = *this; ++t; return *this = t; }
  THRUST_CDNA4_HD value_type operator++(int) { value_type t = *this, old = t; ++t; *this = t; return old; }
  THRUST_CDNA4_HD device_reference& operator--() { value_type t = *this; --t; return *this = t; }
  THRUST_CDNA4_HD value_type operator--(int) { value_type t = *this, old = t; --t; *this = t; return old; }
#define THRUST_CDNA4_REFERENCE_COMPOUND(OP) \
  template <class U> THRUST_CDNA4_HD device_reference& operator OP(const U& r) { value_type t = *this; t OP r; return *this = t; }
  THRUST_CDNA4_REFERENCE_COMPOUND(+=)
  THRUST_CDNA4_REFERENCE_COMPOUND(-=)
  THRUST_CDNA4_REFERENCE_COMPOUND(*=)
  THRUST_CDNA4_REFERENCE_COMPOUND(/=)
  THRUST_CDNA4_REFERENCE_COMPOUND(%=)
  THRUST_CDNA4_REFERENCE_COMPOUND(<<=)
  THRUST_CDNA4_REFERENCE_COMPOUND(>>=)
  THRUST_CDNA4_REFERENCE_COMPOUND(&=)
  THRUST_CDNA4_REFERENCE_COMPOUND(|=)
  THRUST_CDNA4_REFERENCE_COMPOUND(^=)
#undef THRUST_CDNA4_REFERENCE_COMPOUND
  THRUST_CDNA4_HD void swap(device_reference& o) { value_type a = *this, b = o; *this = b; o = a; }

 private:
  T* p_;
};

template <class T>
class device_ptr {
 public:
  typedef std::random_access_iterator_tag iterator_category;
  typedef typename std::remove_const<T>::type value_type;
  typedef std::ptrdiff_t difference_type;
  typedef device_ptr pointer;
  typedef device_reference<T> reference;
  typedef system::cdna4::tag system_tag;

  THRUST_CDNA4_HD device_ptr() : p_(nullptr) {}
  THRUST_CDNA4_HD device_ptr(std::nullptr_t) : p_(nullptr) {}  // a NullablePointer, as std::unique_ptr and allocators need
  THRUST_CDNA4_HD explicit device_ptr(T* p) : p_(p) {}
  THRUST_CDNA4_HD explicit operator bool() const { return p_ != nullptr; }
  THRUST_CDNA4_HD friend bool operator==(device_ptr a, std::nullptr_t) { return a.p_ == nullptr; }
  THRUST_CDNA4_HD friend bool operator==(std::nullptr_t, device_ptr a) { return a.p_ == nullptr; }
  THRUST_CDNA4_HD friend bool operator!=(device_ptr a, std::nullptr_t) { return a.p_ != nullptr; }
  THRUST_CDNA4_HD friend bool operator!=(std::nullptr_t, device_ptr a) { return a.p_ != nullptr; }
  template <class U, class = typename std::enable_if<std::is_convertible<U*, T*>::value>::type>
  THRUST_CDNA4_HD device_ptr(const device_ptr<U>& o) : p_(o.get()) {}
  THRUST_CDNA4_HD T* get() const { return p_; }
  // member access: in a kernel, and on the host for memory the host can address (universal memory)
  THRUST_CDNA4_HD T* operator->() const { return p_; }
  THRUST_CDNA4_HD reference operator*() const { return reference(p_); }
  THRUST_CDNA4_HD reference operator[](difference_type i) const { return reference(p_ + i); }
  THRUST_CDNA4_HD device_ptr& operator++() { ++p_; return *this; }
  THRUST_CDNA4_HD device_ptr operator++(int) { device_ptr t(*this); ++p_; return t; }
  THRUST_CDNA4_HD device_ptr& operator--() { --p_; return *this; }
  THRUST_CDNA4_HD device_ptr operator--(int) { device_ptr t(*this); --p_; return t; }
  THRUST_CDNA4_HD device_ptr& operator+=(difference_type d) { p_ += d; return *this; }
  THRUST_CDNA4_HD device_ptr& operator-=(difference_type d) { p_ -= d; return *this; }
  THRUST_CDNA4_HD friend device_ptr operator+(device_ptr a, difference_type d) { return device_ptr(a.p_ + d); }
  THRUST_CDNA4_HD friend device_ptr operator+(difference_type d, device_ptr a) { return device_ptr(a.p_ + d); }
  THRUST_CDNA4_HD friend device_ptr operator-(device_ptr a, difference_type d) { return device_ptr(a.p_ - d); }
  THRUST_CDNA4_HD friend difference_type operator-(device_ptr a, device_ptr b) { return a.p_ - b.p_; }
  THRUST_CDNA4_HD friend bool operator==(device_ptr a, device_ptr b) { return a.p_ == b.p_; }
  THRUST_CDNA4_HD friend bool operator!=(device_ptr a, device_ptr b) { return a.p_ != b.p_; }
  THRUST_CDNA4_HD friend bool operator<(device_ptr a, device_ptr b) { return a.p_ < b.p_; }
  THRUST_CDNA4_HD friend bool operator>(device_ptr a, device_ptr b) { return a.p_ > b.p_; }
  THRUST_CDNA4_HD friend bool operator<=(device_ptr a, device_ptr b) { return a.p_ <= b.p_; }
  THRUST_CDNA4_HD friend bool operator>=(device_ptr a, device_ptr b) { return a.p_ >= b.p_; }

 private:
  T* p_;
};

template <class T> THRUST_CDNA4_HD inline void swap(device_reference<T> a, device_reference<T> b) { a.swap(b); }
// streamed as the element's value and as the raw address (thrust/device_reference.h:975, thrust/device_ptr.h:170)
template <class Ch, class Tr, class T>
std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const device_reference<T>& r) {
  return os << static_cast<typename device_reference<T>::value_type>(r);
}
template <class Ch, class Tr, class T>
std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const device_ptr<T>& p) {
  return os << static_cast<const void*>(p.get());
}
template <class T> THRUST_CDNA4_HD inline device_ptr<T> device_pointer_cast(T* p) { return device_ptr<T>(p); }
template <class T> THRUST_CDNA4_HD inline device_ptr<T> device_pointer_cast(device_ptr<T> p) { return p; }
template <class T> THRUST_CDNA4_HD inline T* raw_pointer_cast(device_ptr<T> p) { return p.get(); }
template <class T> THRUST_CDNA4_HD inline T* raw_pointer_cast(T* p) { return p; }

// Cached, stream-ordered device allocation (thrust/device_malloc.h, device_free.h).
template <class T> inline device_ptr<T> device_malloc(std::size_t n) {
  return device_ptr<T>(static_cast<T*>(system::cdna4::detail::malloc_bytes(n * sizeof(T), nullptr)));
}
template <class T> inline void device_free(device_ptr<T> p) { system::cdna4::detail::free_bytes(p.get(), nullptr); }

namespace system { namespace cdna4 { namespace detail {
// Contiguous device iterators are unwrapped to raw pointers before the C ABI is called
// (thrust/type_traits/is_contiguous_iterator.h:246-, try_unwrap_contiguous_iterator).
// An iterator class says which memory it walks either by a partial specialisation below or by a
// nested typedef `thrust_system_is_device` (std::true_type / std::false_type), which is what
// thrust::iterator_facade and iterator_adaptor define; or by an iterator_category derived from one
// of thrust's *_device_iterator_tag types.
struct device_category_marker {};
template <class It, class = void> struct declares_device_iterator : std::false_type {};
template <class It> struct declares_device_iterator<It, typename std::enable_if<It::thrust_system_is_device::value || !It::thrust_system_is_device::value>::type>
    : It::thrust_system_is_device {};
template <class It, class = void> struct has_device_category : std::false_type {};
template <class It> struct has_device_category<It, typename std::enable_if<std::is_base_of<device_category_marker, typename It::iterator_category>::value>::type>
    : std::true_type {};
template <class It> struct is_device_iterator { static constexpr bool value = declares_device_iterator<It>::value || has_device_category<It>::value; };
template <class T> struct is_device_iterator<T*> { static constexpr bool value = false; };
template <class T> struct is_device_iterator<thrust::device_ptr<T>> { static constexpr bool value = true; };
// Iterators that walk no memory — counting, constant, discard, and adaptors over nothing else —
// belong to any system (thrust/iterator/detail/any_system_tag.h:27-38): they count as device
// iterators, and next to a range in memory they follow that range's system.
template <class It> struct is_any_system_iterator : std::false_type {};
template <class T, bool = std::is_pointer<T>::value, class = void> struct is_iterator_type : std::false_type {};
template <class T> struct is_iterator_type<T, true, void> : std::is_object<typename std::remove_pointer<T>::type> {};
template <class T> struct is_iterator_type<T, false, typename std::conditional<false, typename std::iterator_traits<T>::iterator_category, void>::type> : std::true_type {};
// The system that an algorithm called without a policy runs on, from all of its argument types
// (thrust/detail/generic/select_system.inl:60-170): arguments that are no iterators, and iterators
// of any system, have no say; the first other iterator decides; with none, the device.
template <class... Ts> struct runs_on_device : std::true_type {};
template <class T, class... R> struct runs_on_device<T, R...>
    : std::conditional<!is_iterator_type<T>::value || is_any_system_iterator<T>::value, runs_on_device<R...>,
                       std::integral_constant<bool, is_device_iterator<T>::value>>::type {};
template <class... Ts> struct all_any_system : std::true_type {};
template <class T, class... R> struct all_any_system<T, R...> : std::integral_constant<bool, is_any_system_iterator<T>::value && all_any_system<R...>::value> {};
}}}  // namespace system::cdna4::detail
}  // namespace thrust
