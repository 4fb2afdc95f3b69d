// thrust::detail::normal_iterator<Pointer> (thrust/iterator/detail/normal_iterator.h:35-75): the
// random-access iterator of thrust::host_vector — a pointer in a class of thrust's own, so that
// argument-dependent lookup on a host_vector's iterators finds thrust's functions and not std's.
#pragma once
#include <cstddef>
#include <iterator>
#include <type_traits>
#include <thrust/detail/hd.h>
namespace thrust {
namespace detail {
template <class Pointer>
class normal_iterator {
 public:
  typedef typename std::iterator_traits<Pointer>::value_type value_type;
  typedef typename std::iterator_traits<Pointer>::reference reference;
  typedef typename std::iterator_traits<Pointer>::difference_type difference_type;
  typedef Pointer pointer;
  typedef std::random_access_iterator_tag iterator_category;
  typedef std::false_type thrust_system_is_device;

  THRUST_CDNA4_HD normal_iterator() : p_() {}
  THRUST_CDNA4_HD explicit normal_iterator(Pointer p) : p_(p) {}
  // iterator -> const_iterator
  template <class Other, class = typename std::enable_if<std::is_convertible<Other, Pointer>::value>::type>
  THRUST_CDNA4_HD normal_iterator(const normal_iterator<Other>& o) : p_(o.base()) {}

  THRUST_CDNA4_HD Pointer base() const { return p_; }
  THRUST_CDNA4_HD reference operator*() const { return *p_; }
  THRUST_CDNA4_HD Pointer operator->() const { return p_; }
  THRUST_CDNA4_HD reference operator[](difference_type n) const { return p_[n]; }
  THRUST_CDNA4_HD normal_iterator& operator++() { ++p_; return *this; }
  THRUST_CDNA4_HD normal_iterator operator++(int) { normal_iterator t(*this); ++p_; return t; }
  THRUST_CDNA4_HD normal_iterator& operator--() { --p_; return *this; }
  THRUST_CDNA4_HD normal_iterator operator--(int) { normal_iterator t(*this); --p_; return t; }
  THRUST_CDNA4_HD normal_iterator& operator+=(difference_type n) { p_ += n; return *this; }
  THRUST_CDNA4_HD normal_iterator& operator-=(difference_type n) { p_ -= n; return *this; }
  THRUST_CDNA4_HD normal_iterator operator+(difference_type n) const { return normal_iterator(p_ + n); }
  THRUST_CDNA4_HD normal_iterator operator-(difference_type n) const { return normal_iterator(p_ - n); }
  THRUST_CDNA4_HD friend normal_iterator operator+(difference_type n, const normal_iterator& it) { return normal_iterator(it.p_ + n); }

 private:
  Pointer p_;
};
template <class P, class Q>
THRUST_CDNA4_HD auto operator-(const normal_iterator<P>& a, const normal_iterator<Q>& b) -> decltype(a.base() - b.base()) { return a.base() - b.base(); }
template <class P, class Q> THRUST_CDNA4_HD bool operator==(const normal_iterator<P>& a, const normal_iterator<Q>& b) { return a.base() == b.base(); }
template <class P, class Q> THRUST_CDNA4_HD bool operator!=(const normal_iterator<P>& a, const normal_iterator<Q>& b) { return a.base() != b.base(); }
template <class P, class Q> THRUST_CDNA4_HD bool operator<(const normal_iterator<P>& a, const normal_iterator<Q>& b) { return a.base() < b.base(); }
template <class P, class Q> THRUST_CDNA4_HD bool operator>(const normal_iterator<P>& a, const normal_iterator<Q>& b) { return a.base() > b.base(); }
template <class P, class Q> THRUST_CDNA4_HD bool operator<=(const normal_iterator<P>& a, const normal_iterator<Q>& b) { return a.base() <= b.base(); }
template <class P, class Q> THRUST_CDNA4_HD bool operator>=(const normal_iterator<P>& a, const normal_iterator<Q>& b) { return a.base() >= b.base(); }
template <class Pointer> THRUST_CDNA4_HD normal_iterator<Pointer> make_normal_iterator(Pointer p) { return normal_iterator<Pointer>(p); }
}  // namespace detail
}  // namespace thrust
