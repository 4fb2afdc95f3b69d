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
// The arithmetic, comparison, logical and bitwise function objects (thrust/functional.h:129-1130), each
// with the argument / result typedefs of an adaptable function object and a transparent form
// (thrust::plus<> etc.) that deduces its types per call.
#define THRUST_CDNA4_BINARY_FUNCTOR(NAME, RESULT, EXPR)                                                                   \
  template <class T = void> struct NAME {                                                                                \
    typedef T first_argument_type;                                                                                       \
    typedef T second_argument_type;                                                                                      \
    typedef RESULT result_type;                                                                                          \
    THRUST_CDNA4_HD constexpr RESULT operator()(const T& a, const T& b) const { return EXPR; }                            \
  };                                                                                                                     \
  template <> struct NAME<void> {                                                                                        \
    typedef void is_transparent;                                                                                         \
    template <class A, class B> THRUST_CDNA4_HD constexpr auto operator()(const A& a, const B& b) const -> decltype(EXPR) { return EXPR; } \
  };
#define THRUST_CDNA4_UNARY_FUNCTOR(NAME, RESULT, EXPR)                                                                    \
  template <class T = void> struct NAME {                                                                                \
    typedef T argument_type;                                                                                             \
    typedef RESULT result_type;                                                                                          \
    THRUST_CDNA4_HD constexpr RESULT operator()(const T& a) const { return EXPR; }                                        \
  };                                                                                                                     \
  template <> struct NAME<void> {                                                                                        \
    typedef void is_transparent;                                                                                         \
    template <class A> THRUST_CDNA4_HD constexpr auto operator()(const A& a) const -> decltype(EXPR) { return EXPR; }      \
  };
THRUST_CDNA4_BINARY_FUNCTOR(plus, T, a + b)
THRUST_CDNA4_BINARY_FUNCTOR(minus, T, a - b)
THRUST_CDNA4_BINARY_FUNCTOR(multiplies, T, a * b)
THRUST_CDNA4_BINARY_FUNCTOR(divides, T, a / b)
THRUST_CDNA4_BINARY_FUNCTOR(modulus, T, a % b)
THRUST_CDNA4_UNARY_FUNCTOR(negate, T, -a)
THRUST_CDNA4_UNARY_FUNCTOR(square, T, a * a)
THRUST_CDNA4_BINARY_FUNCTOR(equal_to, bool, a == b)
THRUST_CDNA4_BINARY_FUNCTOR(not_equal_to, bool, a != b)
THRUST_CDNA4_BINARY_FUNCTOR(greater, bool, a > b)
THRUST_CDNA4_BINARY_FUNCTOR(less, bool, a < b)
THRUST_CDNA4_BINARY_FUNCTOR(greater_equal, bool, a >= b)
THRUST_CDNA4_BINARY_FUNCTOR(less_equal, bool, a <= b)
THRUST_CDNA4_BINARY_FUNCTOR(logical_and, bool, a && b)
THRUST_CDNA4_BINARY_FUNCTOR(logical_or, bool, a || b)
THRUST_CDNA4_UNARY_FUNCTOR(logical_not, bool, !a)
THRUST_CDNA4_BINARY_FUNCTOR(bit_and, T, a & b)
THRUST_CDNA4_BINARY_FUNCTOR(bit_or, T, a | b)
THRUST_CDNA4_BINARY_FUNCTOR(bit_xor, T, a ^ b)
#undef THRUST_CDNA4_BINARY_FUNCTOR
#undef THRUST_CDNA4_UNARY_FUNCTOR
// maximum / minimum return one of their arguments (thrust/functional.h:1196-1284): the first of two
// equivalent ones for minimum, the first for maximum as well (a < b ? b : a)
template <class T = void> struct maximum {
  typedef T first_argument_type; typedef T second_argument_type; typedef T result_type;
  THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a < b ? b : a; }
};
template <class T = void> struct minimum {
  typedef T first_argument_type; typedef T second_argument_type; typedef T result_type;
  THRUST_CDNA4_HD constexpr T operator()(const T& a, const T& b) const { return a < b ? a : b; }
};
template <> struct maximum<void> { typedef void is_transparent; template <class A> THRUST_CDNA4_HD constexpr A operator()(const A& a, const A& b) const { return a < b ? b : a; } };
template <> struct minimum<void> { typedef void is_transparent; template <class A> THRUST_CDNA4_HD constexpr A operator()(const A& a, const A& b) const { return a < b ? a : b; } };
template <class T = void> struct identity {
  typedef T argument_type; typedef T result_type;
  THRUST_CDNA4_HD constexpr const T& operator()(const T& a) const { return a; }
};
template <> struct identity<void> { typedef void is_transparent; template <class A> THRUST_CDNA4_HD constexpr const A& operator()(const A& a) const { return a; } };
// project1st / project2nd return one of their two arguments (thrust/functional.h:1303-1396)
template <class T1 = void, class T2 = void> struct project1st {
  typedef T1 first_argument_type; typedef T2 second_argument_type; typedef T1 result_type;
  THRUST_CDNA4_HD constexpr const T1& operator()(const T1& a, const T2&) const { return a; }
};
template <> struct project1st<void, void> { typedef void is_transparent; template <class A, class B> THRUST_CDNA4_HD constexpr const A& operator()(const A& a, const B&) const { return a; } };
template <class T1 = void, class T2 = void> struct project2nd {
  typedef T1 first_argument_type; typedef T2 second_argument_type; typedef T2 result_type;
  THRUST_CDNA4_HD constexpr const T2& operator()(const T1&, const T2& b) const { return b; }
};
template <> struct project2nd<void, void> { typedef void is_transparent; template <class A, class B> THRUST_CDNA4_HD constexpr const B& operator()(const A&, const B& b) const { return b; } };
// negators (thrust/functional.h:1411-1529): unary_negate / not1 and binary_negate / not2 for adaptable
// predicates, not_fn for any callable
template <class Predicate> struct unary_negate : unary_function<typename Predicate::argument_type, bool> {
  THRUST_CDNA4_HD explicit unary_negate(Predicate p) : pred(p) {}
  THRUST_CDNA4_HD bool operator()(const typename Predicate::argument_type& x) { return !pred(x); }
  Predicate pred;
};
template <class Predicate> THRUST_CDNA4_HD unary_negate<Predicate> not1(const Predicate& pred) { return unary_negate<Predicate>(pred); }
template <class Predicate> struct binary_negate : binary_function<typename Predicate::first_argument_type, typename Predicate::second_argument_type, bool> {
  THRUST_CDNA4_HD explicit binary_negate(Predicate p) : pred(p) {}
  THRUST_CDNA4_HD bool operator()(const typename Predicate::first_argument_type& x, const typename Predicate::second_argument_type& y) { return !pred(x, y); }
  Predicate pred;
};
template <class Predicate> THRUST_CDNA4_HD binary_negate<Predicate> not2(const Predicate& pred) { return binary_negate<Predicate>(pred); }
namespace detail {
template <class F> struct not_fun_t {
  F f;
  template <class... Ts> THRUST_CDNA4_HD auto operator()(Ts&&... ts) -> decltype(!f(static_cast<Ts&&>(ts)...)) { return !f(static_cast<Ts&&>(ts)...); }
  template <class... Ts> THRUST_CDNA4_HD auto operator()(Ts&&... ts) const -> decltype(!f(static_cast<Ts&&>(ts)...)) { return !f(static_cast<Ts&&>(ts)...); }
};
}  // namespace detail
template <class F> THRUST_CDNA4_HD detail::not_fun_t<F> not_fn(F f) { return detail::not_fun_t<F>{f}; }

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
