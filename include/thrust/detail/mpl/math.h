// <thrust/detail/mpl/math.h>: compile-time integer arithmetic (thrust/detail/mpl/math.h:30-170).
#pragma once
#include <thrust/detail/config.h>
namespace thrust { namespace detail { namespace mpl { namespace math {
namespace detail {
constexpr unsigned floor_log2(unsigned long long n) { return n <= 1 ? 0u : 1u + floor_log2(n / 2); }
}  // namespace detail
template <unsigned long long N> struct log2 { static_assert(N != 0, "log2 of zero"); static const unsigned int value = detail::floor_log2(N); };
template <class T, T a, T b> struct min { static const T value = a < b ? a : b; };
template <class T, T a, T b> struct max { static const T value = a > b ? a : b; };
template <class R, R a, R b> struct mul { static const R value = a * b; };
template <class R, R a, R b> struct mod { static const R value = a % b; };
template <class R, R a, R b> struct div { static const R value = a / b; };
template <class R, R a, R b> struct geq { static const bool value = a >= b; };
template <class R, R a, R b> struct lt { static const bool value = a < b; };
template <class R, R a, R b> struct gt { static const bool value = a > b; };
template <bool a, bool b> struct or_ { static const bool value = a || b; };
template <class R, R a, R b> struct bit_and { static const R value = a & b; };
template <class R, R a, R b> struct plus { static const R value = a + b; };
template <class R, R a, R b> struct minus { static const R value = a - b; };
template <class R, R a, R b> struct equal { static const bool value = a == b; };
template <class R, R a> struct is_odd { static const bool value = (a & 1) != 0; };
}}}}  // namespace thrust::detail::mpl::math
