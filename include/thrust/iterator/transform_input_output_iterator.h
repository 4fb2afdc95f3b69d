// thrust::transform_input_output_iterator (thrust/iterator/transform_input_output_iterator.h):
// reading element n gives input_function(base[n]); assigning x stores output_function(x) there.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/iterator/detail/fancy_base.h>

namespace thrust {
namespace detail {
template <class InF, class OutF, class It> struct transform_io_proxy {
  typedef typename std::decay<decltype(std::declval<InF&>()(std::declval<typename std::iterator_traits<It>::value_type>()))>::type value;
  It it; InF in; OutF out;
  THRUST_CDNA4_HD operator value() const { return in(*it); }
  template <class T> THRUST_CDNA4_HD const transform_io_proxy& operator=(const T& x) const {
    *it = out(x);
    return *this;
  }
  THRUST_CDNA4_HD const transform_io_proxy& operator=(const transform_io_proxy& o) const {
    *it = out(static_cast<value>(o));
    return *this;
  }
};
}  // namespace detail
template <class InF, class OutF, class It>
class transform_input_output_iterator
    : public detail::fancy_base<transform_input_output_iterator<InF, OutF, It>, detail::transform_io_proxy<InF, OutF, It>> {
 public:
  typedef detail::transform_io_proxy<InF, OutF, It> reference;
  typedef typename reference::value value_type;
  transform_input_output_iterator() : it_(), in_(), out_() {}
  THRUST_CDNA4_HD transform_input_output_iterator(It it, InF in, OutF out) : it_(it), in_(in), out_(out) {}
  THRUST_CDNA4_HD reference at(std::ptrdiff_t n) const { return reference{it_ + n, in_, out_}; }
  THRUST_CDNA4_HD void advance(std::ptrdiff_t n) { it_ += n; }
  THRUST_CDNA4_HD std::ptrdiff_t distance_to(const transform_input_output_iterator& o) const { return o.it_ - it_; }
  THRUST_CDNA4_HD It base() const { return it_; }
  THRUST_CDNA4_HD InF input_function() const { return in_; }
  THRUST_CDNA4_HD OutF output_function() const { return out_; }
 private:
  It it_;
  mutable InF in_;
  mutable OutF out_;
};
template <class InF, class OutF, class It>
THRUST_CDNA4_HD transform_input_output_iterator<InF, OutF, It> make_transform_input_output_iterator(It it, InF in, OutF out) {
  return transform_input_output_iterator<InF, OutF, It>(it, in, out);
}
namespace system { namespace cdna4 { namespace detail {
template <class InF, class OutF, class It> struct is_device_iterator<thrust::transform_input_output_iterator<InF, OutF, It>> : is_device_iterator<It> {};
template <class InF, class OutF, class It> struct is_any_system_iterator<thrust::transform_input_output_iterator<InF, OutF, It>> : is_any_system_iterator<It> {};
}}}
namespace detail {
template <class InF, class OutF, class It> struct unwrap_iterator<thrust::transform_input_output_iterator<InF, OutF, It>> {
  typedef thrust::transform_input_output_iterator<InF, OutF, typename unwrap_iterator<It>::type> type;
  static type apply(const thrust::transform_input_output_iterator<InF, OutF, It>& it) {
    return type(unwrap(it.base()), it.input_function(), it.output_function());
  }
};
}  // namespace detail
}  // namespace thrust
