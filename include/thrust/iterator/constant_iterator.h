// thrust::constant_iterator (thrust/iterator/constant_iterator.h): every element is the value.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
template <class T>
class constant_iterator : public detail::fancy_base<constant_iterator<T>, T> {
 public:
  typedef T value_type;
  typedef T reference;
  constant_iterator() : v_(), pos_(0) {}
  THRUST_CDNA4_HD explicit constant_iterator(T v, std::ptrdiff_t pos = 0) : v_(v), pos_(pos) {}
  THRUST_CDNA4_HD T at(std::ptrdiff_t) const { return v_; }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { pos_ += n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const constant_iterator& o) const { return o.pos_ - pos_; }
  THRUST_CDNA4_HD const T& value() const { return v_; }  // thrust/iterator/constant_iterator.h:173
  THRUST_CDNA4_HD counting_iterator<std::ptrdiff_t> base() const { return counting_iterator<std::ptrdiff_t>(pos_); }  // its position
 private:
  T v_;
  std::ptrdiff_t pos_;
};
template <class T> THRUST_CDNA4_HD constant_iterator<T> make_constant_iterator(T v) { return constant_iterator<T>(v); }
namespace system { namespace cdna4 { namespace detail {
template <class T> struct is_device_iterator<thrust::constant_iterator<T>> { static constexpr bool value = true; };
template <class T> struct is_any_system_iterator<thrust::constant_iterator<T>> : std::true_type {};
}}}
}  // namespace thrust
