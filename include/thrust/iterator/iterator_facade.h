// thrust::iterator_facade and iterator_core_access (thrust/iterator/iterator_facade.h): the full
// iterator interface from a few core functions of the derived class — dereference(), increment(),
// decrement(), advance(n), equal(other), distance_to(other) — reached through
// iterator_core_access so that they may be private.  System says which memory the iterator walks
// (thrust::device_system_tag or host_system_tag): the algorithms dispatch on it.
#pragma once
#include <cstddef>
#include <iterator>
#include <type_traits>
#include <thrust/detail/hd.h>
#include <thrust/execution_policy.h>
#include <thrust/iterator/detail/fancy_base.h>
#include <thrust/iterator/iterator_categories.h>
namespace thrust {
class iterator_core_access {
 public:
  template <class F> THRUST_CDNA4_HD static typename F::reference dereference(const F& f) { return f.dereference(); }
  template <class F> THRUST_CDNA4_HD static void increment(F& f) { f.increment(); }
  template <class F> THRUST_CDNA4_HD static void decrement(F& f) { f.decrement(); }
  template <class F> THRUST_CDNA4_HD static void advance(F& f, typename F::difference_type n) { f.advance(n); }
  template <class F1, class F2> THRUST_CDNA4_HD static bool equal(const F1& a, const F2& b) { return a.equal(b); }
  template <class F1, class F2> THRUST_CDNA4_HD static typename F1::difference_type distance_from(const F1& a, const F2& b) { return -a.distance_to(b); }
  template <class F1, class F2> THRUST_CDNA4_HD static typename F1::difference_type distance_to(const F1& a, const F2& b) { return a.distance_to(b); }
};

template <class Derived, class Value, class System, class Traversal, class Reference, class Difference = std::ptrdiff_t>
class iterator_facade {
  THRUST_CDNA4_HD Derived& derived() { return *static_cast<Derived*>(this); }
  THRUST_CDNA4_HD const Derived& derived() const { return *static_cast<const Derived*>(this); }
 public:
  typedef typename std::remove_const<Value>::type value_type;
  typedef Reference reference;
  typedef void pointer;
  typedef Difference difference_type;
  typedef std::integral_constant<bool, std::is_convertible<System, device_system_tag>::value> thrust_system_is_device;
  typedef typename detail::category_of_traversal<Traversal, thrust_system_is_device::value>::type iterator_category;

  THRUST_CDNA4_HD reference operator*() const { return iterator_core_access::dereference(derived()); }
  THRUST_CDNA4_HD reference operator[](difference_type n) const { return *(derived() + n); }
  THRUST_CDNA4_HD Derived& operator++() { iterator_core_access::increment(derived()); return derived(); }
  THRUST_CDNA4_HD Derived operator++(int) { Derived t(derived()); iterator_core_access::increment(derived()); return t; }
  THRUST_CDNA4_HD Derived& operator--() { iterator_core_access::decrement(derived()); return derived(); }
  THRUST_CDNA4_HD Derived operator--(int) { Derived t(derived()); iterator_core_access::decrement(derived()); return t; }
  THRUST_CDNA4_HD Derived& operator+=(difference_type n) { iterator_core_access::advance(derived(), n); return derived(); }
  THRUST_CDNA4_HD Derived& operator-=(difference_type n) { iterator_core_access::advance(derived(), -n); return derived(); }
  THRUST_CDNA4_HD Derived operator-(difference_type n) const { Derived t(derived()); return t -= n; }
  THRUST_CDNA4_HD friend Derived operator+(const Derived& a, difference_type n) { Derived t(a); return t += n; }
  THRUST_CDNA4_HD friend Derived operator+(difference_type n, const Derived& a) { Derived t(a); return t += n; }
  THRUST_CDNA4_HD friend difference_type operator-(const Derived& a, const Derived& b) { return iterator_core_access::distance_to(b, a); }
  THRUST_CDNA4_HD friend bool operator==(const Derived& a, const Derived& b) { return iterator_core_access::equal(a, b); }
  THRUST_CDNA4_HD friend bool operator!=(const Derived& a, const Derived& b) { return !iterator_core_access::equal(a, b); }
  THRUST_CDNA4_HD friend bool operator<(const Derived& a, const Derived& b) { return iterator_core_access::distance_to(a, b) > 0; }
  THRUST_CDNA4_HD friend bool operator>(const Derived& a, const Derived& b) { return iterator_core_access::distance_to(a, b) < 0; }
  THRUST_CDNA4_HD friend bool operator<=(const Derived& a, const Derived& b) { return iterator_core_access::distance_to(a, b) >= 0; }
  THRUST_CDNA4_HD friend bool operator>=(const Derived& a, const Derived& b) { return iterator_core_access::distance_to(a, b) <= 0; }
};
}  // namespace thrust
