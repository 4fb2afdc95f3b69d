// Random-access boilerplate shared by the fancy iterators (thrust/iterator/iterator_facade.h):
// a derived iterator supplies at(n) — the element n positions from here — advance(n),
// distance_to(other) and the typedefs value_type / reference; Reference is what at() returns.
#pragma once
#include <cstddef>
#include <iterator>
#include <thrust/functional.h>
#include <thrust/iterator/iterator_traits.h>

namespace thrust {
// a template argument left to its default (thrust/iterator/detail/use_default.h)
struct use_default {};
namespace detail {
template <class Derived, class Reference>
struct fancy_base {
  typedef std::random_access_iterator_tag iterator_category;
  typedef std::ptrdiff_t difference_type;
  typedef void pointer;
  THRUST_CDNA4_HD Derived& self() { return static_cast<Derived&>(*this); }
  THRUST_CDNA4_HD const Derived& self() const { return static_cast<const Derived&>(*this); }
  THRUST_CDNA4_HD Reference operator*() const { return self().at(0); }
  THRUST_CDNA4_HD Reference operator[](difference_type n) const { return self().at(n); }
  THRUST_CDNA4_HD Derived& operator++() { self().advance(1); return self(); }
  THRUST_CDNA4_HD Derived operator++(int) { Derived t(self()); self().advance(1); return t; }
  THRUST_CDNA4_HD Derived& operator--() { self().advance(-1); return self(); }
  THRUST_CDNA4_HD Derived operator--(int) { Derived t(self()); self().advance(-1); return t; }
  THRUST_CDNA4_HD Derived& operator+=(difference_type n) { self().advance(n); return self(); }
  THRUST_CDNA4_HD Derived& operator-=(difference_type n) { self().advance(-n); return self(); }
  THRUST_CDNA4_HD friend Derived operator+(const Derived& a, difference_type n) { Derived t(a); t.advance(n); return t; }
  THRUST_CDNA4_HD friend Derived operator+(difference_type n, const Derived& a) { Derived t(a); t.advance(n); return t; }
  THRUST_CDNA4_HD friend Derived operator-(const Derived& a, difference_type n) { Derived t(a); t.advance(-n); return t; }
  THRUST_CDNA4_HD friend difference_type operator-(const Derived& a, const Derived& b) { return b.distance_to(a); }
  THRUST_CDNA4_HD friend bool operator==(const Derived& a, const Derived& b) { return b.distance_to(a) == 0; }
  THRUST_CDNA4_HD friend bool operator!=(const Derived& a, const Derived& b) { return b.distance_to(a) != 0; }
  THRUST_CDNA4_HD friend bool operator<(const Derived& a, const Derived& b) { return a.distance_to(b) > 0; }
  THRUST_CDNA4_HD friend bool operator>(const Derived& a, const Derived& b) { return a.distance_to(b) < 0; }
  THRUST_CDNA4_HD friend bool operator<=(const Derived& a, const Derived& b) { return a.distance_to(b) >= 0; }
  THRUST_CDNA4_HD friend bool operator>=(const Derived& a, const Derived& b) { return a.distance_to(b) <= 0; }
};
}  // namespace detail
}  // namespace thrust
