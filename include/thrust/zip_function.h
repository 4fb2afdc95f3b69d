// thrust::zip_function / make_zip_function (thrust/zip_function.h): adapts an N-ary function to
// take one tuple of N elements, which is what a zip_iterator dereferences to.
#pragma once
#include <utility>
#include <thrust/tuple.h>

namespace thrust {
namespace detail {
template <class F, class Tuple, std::size_t... Is>
THRUST_CDNA4_HD auto zip_apply(F& f, Tuple&& t, std::index_sequence<Is...>) -> decltype(f(thrust::get<Is>(t)...)) {
  return f(thrust::get<Is>(t)...);
}
}  // namespace detail
template <class Function>
class zip_function {
 public:
  zip_function() = default;
  THRUST_CDNA4_HD zip_function(Function f) : f_(f) {}
  template <class Tuple>
  THRUST_CDNA4_HD auto operator()(Tuple&& t) const
      -> decltype(detail::zip_apply(std::declval<Function&>(), t, std::make_index_sequence<tuple_size<typename std::decay<Tuple>::type>::value>())) {
    return detail::zip_apply(f_, t, std::make_index_sequence<tuple_size<typename std::decay<Tuple>::type>::value>());
  }
  THRUST_CDNA4_HD Function& underlying_function() const { return f_; }

 private:
  mutable Function f_;
};
template <class Function>
THRUST_CDNA4_HD zip_function<typename std::decay<Function>::type> make_zip_function(Function&& f) {
  return zip_function<typename std::decay<Function>::type>(static_cast<Function&&>(f));
}
}  // namespace thrust
