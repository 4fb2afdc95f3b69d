// thrust::transform_iterator (thrust/iterator/transform_iterator.h): element n is f(base[n]).
#pragma once
#include <type_traits>
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
namespace detail {
// a functor that hands its argument back (thrust::identity<>) returns the base's proxy reference:
// the element type is then what the proxy stands for
template <class T> struct unproxied { typedef T type; };
template <class U> struct unproxied<thrust::device_reference<U>> { typedef typename std::remove_const<U>::type type; };
template <class F, class It> struct transformed_value {
  typedef typename unproxied<typename std::decay<decltype(std::declval<F&>()(std::declval<typename std::iterator_traits<It>::reference>()))>::type>::type type;
};
}  // namespace detail
namespace detail {
// the element type: named by the user (third or fourth template argument, for functors whose
// result cannot be deduced), else what the functor returns for the base's element
template <class F, class It, class Reference, class Value> struct transform_iterator_value {
  typedef typename std::conditional<
      !std::is_same<Value, use_default>::value, std::decay<Value>,
      typename std::conditional<!std::is_same<Reference, use_default>::value, std::decay<Reference>, transformed_value<F, It>>::type>::type::type type;
};
}  // namespace detail
template <class F, class It, class Reference = use_default, class Value = use_default>
class transform_iterator
    : public detail::fancy_base<transform_iterator<F, It, Reference, Value>, typename detail::transform_iterator_value<F, It, Reference, Value>::type> {
 public:
  typedef typename detail::transform_iterator_value<F, It, Reference, Value>::type value_type;
  typedef value_type reference;
  transform_iterator() : it_(), f_() {}
  THRUST_CDNA4_HD transform_iterator(It it, F f) : it_(it), f_(f) {}
  THRUST_CDNA4_HD value_type at(std::ptrdiff_t n) const { return f_(it_[n]); }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { it_ += n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const transform_iterator& o) const { return o.it_ - it_; }
  THRUST_CDNA4_HD It base() const { return it_; }
  THRUST_CDNA4_HD F functor() const { return f_; }
 private:
  It it_;
  mutable F f_;  // functors with a non-const operator() are accepted, as in the reference
};
template <class F, class It>
THRUST_CDNA4_HD transform_iterator<F, It> make_transform_iterator(It it, F f) { return transform_iterator<F, It>(it, f); }
namespace system { namespace cdna4 { namespace detail {
template <class F, class It, class R, class V> struct is_device_iterator<thrust::transform_iterator<F, It, R, V>> : is_device_iterator<It> {};
template <class F, class It, class R, class V> struct is_any_system_iterator<thrust::transform_iterator<F, It, R, V>> : is_any_system_iterator<It> {};
}}}
namespace detail {
template <class F, class It, class R, class V> struct unwrap_iterator<thrust::transform_iterator<F, It, R, V>> {
  typedef thrust::transform_iterator<F, typename unwrap_iterator<It>::type, R, V> type;
  static type apply(const thrust::transform_iterator<F, It, R, V>& it) { return type(unwrap(it.base()), it.functor()); }
};
}  // namespace detail
}  // namespace thrust
