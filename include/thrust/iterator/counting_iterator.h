// thrust::counting_iterator (thrust/iterator/counting_iterator.h): element n is first + n.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
// System, Traversal and Difference are accepted as in the reference; only a host system tag has an
// effect (the range then counts as a host range).
template <class T, class System = use_default, class Traversal = use_default, class Difference = use_default>
class counting_iterator : public detail::fancy_base<counting_iterator<T, System, Traversal, Difference>, T> {
 public:
  typedef T value_type;
  typedef T reference;
  counting_iterator() : v_() {}
  THRUST_CDNA4_HD explicit counting_iterator(T v) : v_(v) {}
  // the same counter under another system, traversal or difference parameter
  template <class S2, class Tr2, class D2>
  THRUST_CDNA4_HD counting_iterator(const counting_iterator<T, S2, Tr2, D2>& o) : v_(o.base()) {}
  THRUST_CDNA4_HD T at(std::ptrdiff_t n) const { return (T)(v_ + (T)n); }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { v_ = (T)(v_ + (T)n); }
  // signed also for an unsigned counter (thrust/iterator/counting_iterator.h: the difference type of an
  // unsigned counter is a wider signed integer)
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const counting_iterator& o) const { return distance(o.v_, v_, std::is_integral<T>()); }
  THRUST_CDNA4_HD static std::ptrdiff_t distance(const T& to, const T& from, std::true_type) { return (std::ptrdiff_t)to - (std::ptrdiff_t)from; }
  THRUST_CDNA4_HD static std::ptrdiff_t distance(const T& to, const T& from, std::false_type) { return (std::ptrdiff_t)(to - from); }
  THRUST_CDNA4_HD const T& base() const { return v_; }  // the counter (thrust/iterator/iterator_adaptor.h:178)
 private:
  T v_;
};
template <class T> THRUST_CDNA4_HD counting_iterator<T> make_counting_iterator(T v) { return counting_iterator<T>(v); }
namespace system { namespace cdna4 { namespace detail {
template <class T, class S, class Tr, class D> struct is_device_iterator<thrust::counting_iterator<T, S, Tr, D>> {
  static constexpr bool value = !std::is_same<S, thrust::system::cpp::tag>::value;
};
template <class T, class Tr, class D> struct is_any_system_iterator<thrust::counting_iterator<T, use_default, Tr, D>> : std::true_type {};
}}}
}  // namespace thrust
