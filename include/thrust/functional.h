// Function objects the device kernels are specialised on (thrust/functional.h).
#pragma once
#include <functional>
#include <thrust/detail/hd.h>
namespace thrust {
// Empty bases that only carry the argument and result typedefs of an adaptable function object
// (thrust/functional.h:66-126); user functors in existing code derive from them.
template <class Argument, class Result> struct unary_function {
  typedef Argument argument_type;
  typedef Result result_type;
};
template <class Argument1, class Argument2, class Result> struct binary_function {
  typedef Argument1 first_argument_type;
  typedef Argument2 second_argument_type;
  typedef Result result_type;
};
template <class T = void> struct plus { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a + b; } };
template <class T = void> struct multiplies { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a * b; } };
template <class T = void> struct maximum { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a < b ? b : a; } };
template <class T = void> struct minimum { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a < b ? a : b; } };
template <class T = void> struct less { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a < b; } };
template <class T = void> struct greater { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a > b; } };
template <class T = void> struct equal_to { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a == b; } };
template <class T = void> struct minus { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a - b; } };
template <class T = void> struct divides { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a / b; } };
template <class T = void> struct modulus { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a % b; } };
template <class T = void> struct negate { THRUST_CDNA4_HD constexpr T operator()(const T& a) const { return -a; } };
template <class T = void> struct not_equal_to { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a != b; } };
template <class T = void> struct less_equal { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a <= b; } };
template <class T = void> struct greater_equal { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a >= b; } };
template <class T = void> struct logical_and { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a && b; } };
template <class T = void> struct logical_or { THRUST_CDNA4_HD constexpr bool operator()(const T& a, const T& b) const { return a || b; } };
template <class T = void> struct logical_not { THRUST_CDNA4_HD constexpr bool operator()(const T& a) const { return !a; } };
template <class T = void> struct bit_and { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a & b; } };
template <class T = void> struct bit_or { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a | b; } };
template <class T = void> struct bit_xor { THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a ^ b; } };
template <class T = void> struct identity { THRUST_CDNA4_HD constexpr const T& operator()(const T& a) const { return a; } };

// transparent forms (thrust::plus<> etc.)
template <> struct plus<void> { template <class A, class B> THRUST_CDNA4_HD constexpr auto operator()(const A& a, const B& b) const -> decltype(a + b) { return a + b; } };
template <> struct multiplies<void> { template <class A, class B> THRUST_CDNA4_HD constexpr auto operator()(const A& a, const B& b) const -> decltype(a * b) { return a * b; } };
template <> struct maximum<void> { template <class A> THRUST_CDNA4_HD constexpr A operator()(const A& a, const A& b) const { return a < b ? b : a; } };
template <> struct minimum<void> { template <class A> THRUST_CDNA4_HD constexpr A operator()(const A& a, const A& b) const { return a < b ? a : b; } };
template <> struct less<void> { template <class A, class B> THRUST_CDNA4_HD constexpr bool operator()(const A& a, const B& b) const { return a < b; } };
template <> struct greater<void> { template <class A, class B> THRUST_CDNA4_HD constexpr bool operator()(const A& a, const B& b) const { return a > b; } };
template <> struct equal_to<void> { template <class A, class B> THRUST_CDNA4_HD constexpr bool operator()(const A& a, const B& b) const { return a == b; } };

namespace system { namespace cdna4 { namespace detail {
// C-ABI operator code of a functor type, or -1 when no kernel exists for it.
template <class F> struct op_code { static constexpr int value = -1; };
template <class T> struct op_code<thrust::plus<T>> { static constexpr int value = 0; };
template <class T> struct op_code<thrust::multiplies<T>> { static constexpr int value = 1; };
template <class T> struct op_code<thrust::maximum<T>> { static constexpr int value = 2; };
template <class T> struct op_code<thrust::minimum<T>> { static constexpr int value = 3; };
// 0 = ascending (less), 1 = descending (greater), -1 = not a radix-sortable comparator
// (thrust/system/cuda/detail/sort.h:389-395, can_use_primitive_sort).
template <class F> struct order_code { static constexpr int value = -1; };
template <class T> struct order_code<thrust::less<T>> { static constexpr int value = 0; };
template <class T> struct order_code<thrust::greater<T>> { static constexpr int value = 1; };
template <class F> struct is_equal_to { static constexpr bool value = false; };
template <class T> struct is_equal_to<thrust::equal_to<T>> { static constexpr bool value = true; };
}}}  // namespace system::cdna4::detail
}  // namespace thrust
// as in the reference, <thrust/functional.h> brings thrust::tuple and thrust::pair with it
// (placeholder expressions are built on them there)
#include <thrust/pair.h>
#include <thrust/tuple.h>
#include <thrust/detail/placeholders.h>
