// thrust::discard_iterator (thrust/iterator/discard_iterator.h): an output that ignores what is
// assigned to it.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
namespace detail {
struct discard_proxy {
  discard_proxy() = default;
  template <class T> THRUST_CDNA4_HD explicit discard_proxy(const T&) {}  // anything casts to it, and is dropped
  template <class T> THRUST_CDNA4_HD const discard_proxy& operator=(const T&) const { return *this; }
};
}  // namespace detail
// (the System parameter of the reference's template is accepted and ignored: the iterator holds
// no data, so it serves every system)
template <class System = use_default>
class discard_iterator : public detail::fancy_base<discard_iterator<System>, detail::discard_proxy> {
 public:
  typedef detail::discard_proxy value_type;
  typedef detail::discard_proxy reference;
  THRUST_CDNA4_HD explicit discard_iterator(std::ptrdiff_t pos = 0) : pos_(pos) {}
  template <class S2> THRUST_CDNA4_HD discard_iterator(const discard_iterator<S2>& o) : pos_(*o.base()) {}
  THRUST_CDNA4_HD detail::discard_proxy at(std::ptrdiff_t) const { return detail::discard_proxy(); }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { pos_ += n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const discard_iterator& o) const { return o.pos_ - pos_; }
  THRUST_CDNA4_HD counting_iterator<std::ptrdiff_t> base() const { return counting_iterator<std::ptrdiff_t>(pos_); }  // its position
 private:
  std::ptrdiff_t pos_;
};
// positions compare across System parameters
template <class S1, class S2, class = typename std::enable_if<!std::is_same<S1, S2>::value>::type>
THRUST_CDNA4_HD bool operator==(const discard_iterator<S1>& a, const discard_iterator<S2>& b) { return *a.base() == *b.base(); }
template <class S1, class S2, class = typename std::enable_if<!std::is_same<S1, S2>::value>::type>
THRUST_CDNA4_HD bool operator!=(const discard_iterator<S1>& a, const discard_iterator<S2>& b) { return !(a == b); }
THRUST_CDNA4_HD inline discard_iterator<> make_discard_iterator(std::ptrdiff_t pos = 0) { return discard_iterator<>(pos); }
namespace system { namespace cdna4 { namespace detail {
template <class S> struct is_device_iterator<thrust::discard_iterator<S>> { static constexpr bool value = true; };
template <class S> struct is_any_system_iterator<thrust::discard_iterator<S>> : std::true_type {};
}}}
}  // namespace thrust
