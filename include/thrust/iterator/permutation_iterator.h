// thrust::permutation_iterator (thrust/iterator/permutation_iterator.h): element n is
// elements[indices[n]].
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
template <class ElementIt, class IndexIt>
class permutation_iterator : public detail::fancy_base<permutation_iterator<ElementIt, IndexIt>, typename std::iterator_traits<ElementIt>::reference> {
 public:
  typedef typename std::iterator_traits<ElementIt>::value_type value_type;
  typedef typename std::iterator_traits<ElementIt>::reference reference;
  permutation_iterator() : e_(), i_() {}
  THRUST_CDNA4_HD permutation_iterator(ElementIt e, IndexIt i) : e_(e), i_(i) {}
  THRUST_CDNA4_HD reference at(std::ptrdiff_t n) const { return e_[i_[n]]; }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { i_ += n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const permutation_iterator& o) const { return o.i_ - i_; }
  THRUST_CDNA4_HD ElementIt elements() const { return e_; }
  THRUST_CDNA4_HD IndexIt indices() const { return i_; }
  THRUST_CDNA4_HD IndexIt base() const { return i_; }  // the adapted iterator is the index iterator (thrust/iterator/permutation_iterator.h:130)
 private:
  ElementIt e_;
  IndexIt i_;
};
template <class ElementIt, class IndexIt>
THRUST_CDNA4_HD permutation_iterator<ElementIt, IndexIt> make_permutation_iterator(ElementIt e, IndexIt i) {
  return permutation_iterator<ElementIt, IndexIt>(e, i);
}
namespace system { namespace cdna4 { namespace detail {
template <class E, class I> struct is_device_iterator<thrust::permutation_iterator<E, I>> : runs_on_device<E, I> {};
template <class E, class I> struct is_any_system_iterator<thrust::permutation_iterator<E, I>> : all_any_system<E, I> {};
}}}
namespace detail {
template <class E, class I> struct unwrap_iterator<thrust::permutation_iterator<E, I>> {
  typedef thrust::permutation_iterator<typename unwrap_iterator<E>::type, typename unwrap_iterator<I>::type> type;
  static type apply(const thrust::permutation_iterator<E, I>& it) { return type(unwrap(it.elements()), unwrap(it.indices())); }
};
}  // namespace detail
}  // namespace thrust
