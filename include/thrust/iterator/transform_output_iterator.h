// thrust::transform_output_iterator (thrust/iterator/transform_output_iterator.h): assigning x
// to element n stores f(x) in base[n].
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
namespace detail {
template <class F, class It> struct transform_output_proxy {
  It it; F f;
  template <class T> THRUST_CDNA4_HD const transform_output_proxy& operator=(const T& x) const {
    *it = f(x);
    return *this;
  }
};
}  // namespace detail
template <class F, class It>
class transform_output_iterator : public detail::fancy_base<transform_output_iterator<F, It>, detail::transform_output_proxy<F, It>> {
 public:
  typedef void value_type;
  typedef detail::transform_output_proxy<F, It> reference;
  transform_output_iterator() : it_(), f_() {}
  THRUST_CDNA4_HD transform_output_iterator(It it, F f) : it_(it), f_(f) {}
  THRUST_CDNA4_HD reference at(std::ptrdiff_t n) const { return reference{it_ + n, f_}; }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { it_ += n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const transform_output_iterator& o) const { return o.it_ - it_; }
  THRUST_CDNA4_HD It base() const { return it_; }
  THRUST_CDNA4_HD F functor() const { return f_; }
 private:
  It it_;
  mutable F f_;
};
template <class F, class It>
THRUST_CDNA4_HD transform_output_iterator<F, It> make_transform_output_iterator(It it, F f) { return transform_output_iterator<F, It>(it, f); }
namespace system { namespace cdna4 { namespace detail {
template <class F, class It> struct is_device_iterator<thrust::transform_output_iterator<F, It>> : is_device_iterator<It> {};
template <class F, class It> struct is_any_system_iterator<thrust::transform_output_iterator<F, It>> : is_any_system_iterator<It> {};
}}}
namespace detail {
template <class F, class It> struct unwrap_iterator<thrust::transform_output_iterator<F, It>> {
  typedef thrust::transform_output_iterator<F, typename unwrap_iterator<It>::type> type;
  static type apply(const thrust::transform_output_iterator<F, It>& it) { return type(unwrap(it.base()), it.functor()); }
};
}  // namespace detail
}  // namespace thrust
