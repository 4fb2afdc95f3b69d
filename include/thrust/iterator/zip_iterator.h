// thrust::zip_iterator (thrust/iterator/zip_iterator.h): element n is the tuple of the
// component iterators' elements n; dereferencing gives a tuple of their references, which reads
// into and assigns from a tuple of values.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>
#include <thrust/tuple.h>

namespace thrust {
template <class IteratorTuple> class zip_iterator;
template <class... Its>
class zip_iterator<tuple<Its...>> : public detail::fancy_base<zip_iterator<tuple<Its...>>, tuple<typename std::iterator_traits<Its>::reference...>> {
 public:
  typedef tuple<typename std::iterator_traits<Its>::value_type...> value_type;
  typedef tuple<typename std::iterator_traits<Its>::reference...> reference;
  zip_iterator() : its_() {}
  THRUST_CDNA4_HD explicit zip_iterator(const tuple<Its...>& its) : its_(its) {}
  THRUST_CDNA4_HD reference at(std::ptrdiff_t n) const { return at_impl(n, std::index_sequence_for<Its...>()); }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { advance_impl(n, std::index_sequence_for<Its...>()); }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const zip_iterator& o) const { return get<0>(o.its_) - get<0>(its_); }
  THRUST_CDNA4_HD const tuple<Its...>& get_iterator_tuple() const { return its_; }
 private:
  template <std::size_t... Is>
  THRUST_CDNA4_HD reference at_impl(std::ptrdiff_t n, std::index_sequence<Is...>) const { return reference(get<Is>(its_)[n]...); }
  template <std::size_t... Is>
  THRUST_CDNA4_HD void advance_impl(std::ptrdiff_t n, std::index_sequence<Is...>) {
    int unused[] = {0, ((void)(get<Is>(its_) += n), 0)...};
    (void)unused;
  }
  tuple<Its...> its_;
};
template <class... Its>
THRUST_CDNA4_HD zip_iterator<tuple<Its...>> make_zip_iterator(const tuple<Its...>& its) { return zip_iterator<tuple<Its...>>(its); }
template <class... Its, class = typename std::enable_if<(sizeof...(Its) > 1)>::type>
THRUST_CDNA4_HD zip_iterator<tuple<Its...>> make_zip_iterator(Its... its) { return zip_iterator<tuple<Its...>>(tuple<Its...>(its...)); }
namespace system { namespace cdna4 { namespace detail {
template <class It, class... Its> struct is_device_iterator<thrust::zip_iterator<thrust::tuple<It, Its...>>> : runs_on_device<It, Its...> {};
template <class... Its> struct is_any_system_iterator<thrust::zip_iterator<thrust::tuple<Its...>>> : all_any_system<Its...> {};
}}}
namespace detail {
template <class... Its> struct unwrap_iterator<thrust::zip_iterator<thrust::tuple<Its...>>> {
  typedef thrust::zip_iterator<thrust::tuple<typename unwrap_iterator<Its>::type...>> type;
  template <std::size_t... Is>
  static type apply_impl(const thrust::zip_iterator<thrust::tuple<Its...>>& it, std::index_sequence<Is...>) {
    return type(thrust::tuple<typename unwrap_iterator<Its>::type...>(unwrap(thrust::get<Is>(it.get_iterator_tuple()))...));
  }
  static type apply(const thrust::zip_iterator<thrust::tuple<Its...>>& it) { return apply_impl(it, std::index_sequence_for<Its...>()); }
};
}  // namespace detail
}  // namespace thrust
