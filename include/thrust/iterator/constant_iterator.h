// thrust::constant_iterator (thrust/iterator/constant_iterator.h): every element is the value.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
// Incrementable is the type of the position (an index by default); System is accepted as in the
// reference: a host system tag makes the range count as a host range, a device tag as a device range.
template <class T, class Incrementable = use_default, class System = use_default>
class constant_iterator : public detail::fancy_base<constant_iterator<T, Incrementable, System>, T> {
  typedef typename std::conditional<std::is_same<Incrementable, use_default>::value, std::ptrdiff_t, Incrementable>::type index_type;

 public:
  typedef T value_type;
  typedef T reference;
  constant_iterator() : v_(), pos_(0) {}
  THRUST_CDNA4_HD constant_iterator(T v, index_type pos = index_type(0)) : v_(v), pos_(pos) {}
  template <class T2, class I2, class S2, class = typename std::enable_if<std::is_convertible<T2, T>::value>::type>
  THRUST_CDNA4_HD constant_iterator(const constant_iterator<T2, I2, S2>& o) : v_(o.value()), pos_((index_type)*o.base()) {}
  THRUST_CDNA4_HD T at(std::ptrdiff_t) const { return v_; }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { pos_ = (index_type)(pos_ + (index_type)n); }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const constant_iterator& o) const { return (std::ptrdiff_t)(o.pos_ - pos_); }
  THRUST_CDNA4_HD const T& value() const { return v_; }  // thrust/iterator/constant_iterator.h:173
  THRUST_CDNA4_HD counting_iterator<index_type> base() const { return counting_iterator<index_type>(pos_); }  // its position
 private:
  T v_;
  index_type pos_;
};
// positions subtract across index and system parameters
template <class T1, class I1, class S1, class T2, class I2, class S2,
          class = typename std::enable_if<!std::is_same<constant_iterator<T1, I1, S1>, constant_iterator<T2, I2, S2>>::value>::type>
THRUST_CDNA4_HD std::ptrdiff_t operator-(const constant_iterator<T1, I1, S1>& a, const constant_iterator<T2, I2, S2>& b) {
  return (std::ptrdiff_t)*a.base() - (std::ptrdiff_t)*b.base();
}
template <class T> THRUST_CDNA4_HD constant_iterator<T> make_constant_iterator(T v) { return constant_iterator<T>(v); }
template <class T, class I> THRUST_CDNA4_HD constant_iterator<T, I> make_constant_iterator(T v, I pos) { return constant_iterator<T, I>(v, pos); }
namespace system { namespace cdna4 { namespace detail {
template <class T, class I, class S> struct is_device_iterator<thrust::constant_iterator<T, I, S>> {
  static constexpr bool value = !std::is_same<S, thrust::system::cpp::tag>::value;
};
template <class T, class I> struct is_any_system_iterator<thrust::constant_iterator<T, I, use_default>> : std::true_type {};
}}}
}  // namespace thrust
