// <thrust/detail/integer_traits.h>: numeric_limits plus the compile-time constants const_min and
// const_max for the integer types; integer_traits_base serves user specialisations
// (thrust/detail/integer_traits.h:30-130).
#pragma once
#include <thrust/detail/config.h>
#include <climits>
#include <limits>
#include <type_traits>
namespace thrust { namespace detail {
template <class T, T min_val, T max_val> class integer_traits_base {
 public:
  static constexpr bool is_integral = true;
  static constexpr T const_min = min_val;
  static constexpr T const_max = max_val;
};
template <class T, T min_val, T max_val> constexpr T integer_traits_base<T, min_val, max_val>::const_min;
template <class T, T min_val, T max_val> constexpr T integer_traits_base<T, min_val, max_val>::const_max;
namespace integer_traits_detail {
template <class T, bool = std::is_integral<T>::value> class select : public std::numeric_limits<T> {
 public:
  static constexpr bool is_integral = false;
};
template <class T> class select<T, true>
    : public std::numeric_limits<T>,
      public integer_traits_base<T, std::numeric_limits<T>::min(), std::numeric_limits<T>::max()> {
 public:
  using integer_traits_base<T, std::numeric_limits<T>::min(), std::numeric_limits<T>::max()>::is_integral;
};
}  // namespace integer_traits_detail
template <class T> class integer_traits : public integer_traits_detail::select<T> {};
}}  // namespace thrust::detail
