// thrust::reverse_iterator (thrust/iterator/reverse_iterator.h): element n is base[-n - 1].
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
template <class It>
class reverse_iterator : public detail::fancy_base<reverse_iterator<It>, typename std::iterator_traits<It>::reference> {
 public:
  typedef typename std::iterator_traits<It>::value_type value_type;
  typedef typename std::iterator_traits<It>::reference reference;
  reverse_iterator() : it_() {}
  THRUST_CDNA4_HD explicit reverse_iterator(It it) : it_(it) {}
  THRUST_CDNA4_HD reference at(std::ptrdiff_t n) const { return it_[-n - 1]; }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { it_ -= n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const reverse_iterator& o) const { return it_ - o.it_; }
  THRUST_CDNA4_HD It base() const { return it_; }
 private:
  It it_;
};
template <class It> THRUST_CDNA4_HD reverse_iterator<It> make_reverse_iterator(It it) { return reverse_iterator<It>(it); }
namespace system { namespace cdna4 { namespace detail {
template <class It> struct is_device_iterator<thrust::reverse_iterator<It>> : is_device_iterator<It> {};
template <class It> struct is_any_system_iterator<thrust::reverse_iterator<It>> : is_any_system_iterator<It> {};
}}}
namespace detail {
template <class It> struct unwrap_iterator<thrust::reverse_iterator<It>> {
  typedef thrust::reverse_iterator<typename unwrap_iterator<It>::type> type;
  static type apply(const thrust::reverse_iterator<It>& it) { return type(unwrap(it.base())); }
};
}  // namespace detail
}  // namespace thrust
