// thrust::placeholders::_1 ... _10 (thrust/functional.h:1508-, thrust/detail/functional/actor.h):
// small expression templates, so that `a * _1 + _2` is a function object computing a*x + y.
// Operands are placeholders, sub-expressions or plain values (captured by copy); the usual
// arithmetic, comparison, logical and bitwise operators, unary - ! ~, and the assignments
// = += -= *= /= %= &= |= ^= (whose left operand is a placeholder bound to an lvalue) are provided.
#pragma once
#include <cstddef>
#include <type_traits>
#include <utility>
#include <thrust/detail/hd.h>

namespace thrust {
namespace detail { namespace functional {

template <std::size_t I> struct nth_arg {
  template <class A, class... Rest>
  THRUST_CDNA4_HD static constexpr decltype(auto) get(A&&, Rest&&... rest) { return nth_arg<I - 1>::get(static_cast<Rest&&>(rest)...); }
};
template <> struct nth_arg<0> {
  template <class A, class... Rest>
  THRUST_CDNA4_HD static constexpr A&& get(A&& a, Rest&&...) { return static_cast<A&&>(a); }
};

template <std::size_t I> struct argument {
  template <class... A> THRUST_CDNA4_HD constexpr decltype(auto) eval(A&&... a) const { return nth_arg<I>::get(static_cast<A&&>(a)...); }
};
template <class T> struct value {
  T v;
  template <class... A> THRUST_CDNA4_HD constexpr const T& eval(A&&...) const { return v; }
};
template <class Op, class E> struct unary_expr {
  E e;
  template <class... A> THRUST_CDNA4_HD constexpr decltype(auto) eval(A&&... a) const { return Op()(e.eval(static_cast<A&&>(a)...)); }
};
template <class Op, class L, class R> struct binary_expr {
  L l;
  R r;
  template <class... A> THRUST_CDNA4_HD constexpr decltype(auto) eval(A&&... a) const {
    return Op()(l.eval(static_cast<A&&>(a)...), r.eval(static_cast<A&&>(a)...));
  }
};

template <class E> struct actor;
template <class T> struct is_actor : std::false_type {};
template <class E> struct is_actor<actor<E>> : std::true_type {};
// an operand as an expression node: an actor's node, or a captured value
template <class T> struct as_node { typedef value<typename std::decay<T>::type> type; static constexpr type make(const T& t) { return type{t}; } };
template <class E> struct as_node<actor<E>> { typedef E type; THRUST_CDNA4_HD static constexpr const E& make(const actor<E>& a) { return a; } };

#define THRUST_CDNA4_PH_BINARY_OP(NAME, EXPR)                                                      \
  struct NAME {                                                                                     \
    template <class A, class B> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a, B&& b) const { return EXPR; } \
  };
THRUST_CDNA4_PH_BINARY_OP(op_plus, a + b)
THRUST_CDNA4_PH_BINARY_OP(op_minus, a - b)
THRUST_CDNA4_PH_BINARY_OP(op_mul, a * b)
THRUST_CDNA4_PH_BINARY_OP(op_div, a / b)
THRUST_CDNA4_PH_BINARY_OP(op_mod, a % b)
THRUST_CDNA4_PH_BINARY_OP(op_lt, a < b)
THRUST_CDNA4_PH_BINARY_OP(op_gt, a > b)
THRUST_CDNA4_PH_BINARY_OP(op_le, a <= b)
THRUST_CDNA4_PH_BINARY_OP(op_ge, a >= b)
THRUST_CDNA4_PH_BINARY_OP(op_eq, a == b)
THRUST_CDNA4_PH_BINARY_OP(op_ne, a != b)
THRUST_CDNA4_PH_BINARY_OP(op_and, a && b)
THRUST_CDNA4_PH_BINARY_OP(op_or, a || b)
THRUST_CDNA4_PH_BINARY_OP(op_bit_and, a & b)
THRUST_CDNA4_PH_BINARY_OP(op_bit_or, a | b)
THRUST_CDNA4_PH_BINARY_OP(op_bit_xor, a ^ b)
THRUST_CDNA4_PH_BINARY_OP(op_shl, a << b)
THRUST_CDNA4_PH_BINARY_OP(op_shr, a >> b)
THRUST_CDNA4_PH_BINARY_OP(op_assign, a = b)
THRUST_CDNA4_PH_BINARY_OP(op_plus_assign, a += b)
THRUST_CDNA4_PH_BINARY_OP(op_minus_assign, a -= b)
THRUST_CDNA4_PH_BINARY_OP(op_mul_assign, a *= b)
THRUST_CDNA4_PH_BINARY_OP(op_div_assign, a /= b)
THRUST_CDNA4_PH_BINARY_OP(op_mod_assign, a %= b)
THRUST_CDNA4_PH_BINARY_OP(op_and_assign, a &= b)
THRUST_CDNA4_PH_BINARY_OP(op_or_assign, a |= b)
THRUST_CDNA4_PH_BINARY_OP(op_xor_assign, a ^= b)
THRUST_CDNA4_PH_BINARY_OP(op_shl_assign, a <<= b)
THRUST_CDNA4_PH_BINARY_OP(op_shr_assign, a >>= b)
#undef THRUST_CDNA4_PH_BINARY_OP
struct op_negate { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return -a; } };
struct op_not { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return !a; } };
struct op_bit_not { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return ~a; } };
struct op_unary_plus { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return +a; } };
struct op_pre_inc { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return ++a; } };
struct op_pre_dec { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return --a; } };
struct op_post_inc { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return a++; } };
struct op_post_dec { template <class A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&& a) const { return a--; } };

template <class E>
struct actor : E {
  constexpr actor() = default;
  THRUST_CDNA4_HD constexpr actor(const E& e) : E(e) {}
  template <class... A> THRUST_CDNA4_HD constexpr decltype(auto) operator()(A&&... a) const { return this->eval(static_cast<A&&>(a)...); }
#define THRUST_CDNA4_PH_ASSIGN(SYM, OP)                                                            \
  template <class T> THRUST_CDNA4_HD constexpr actor<binary_expr<OP, E, typename as_node<T>::type>> operator SYM(const T& t) const { \
    return actor<binary_expr<OP, E, typename as_node<T>::type>>(binary_expr<OP, E, typename as_node<T>::type>{*this, as_node<T>::make(t)}); \
  }
  THRUST_CDNA4_PH_ASSIGN(=, op_assign)
  THRUST_CDNA4_PH_ASSIGN(+=, op_plus_assign)
  THRUST_CDNA4_PH_ASSIGN(-=, op_minus_assign)
  THRUST_CDNA4_PH_ASSIGN(*=, op_mul_assign)
  THRUST_CDNA4_PH_ASSIGN(/=, op_div_assign)
  THRUST_CDNA4_PH_ASSIGN(%=, op_mod_assign)
  THRUST_CDNA4_PH_ASSIGN(&=, op_and_assign)
  THRUST_CDNA4_PH_ASSIGN(|=, op_or_assign)
  THRUST_CDNA4_PH_ASSIGN(^=, op_xor_assign)
  THRUST_CDNA4_PH_ASSIGN(<<=, op_shl_assign)
  THRUST_CDNA4_PH_ASSIGN(>>=, op_shr_assign)
#undef THRUST_CDNA4_PH_ASSIGN
};

template <class L, class R> struct either_is_actor
    : std::integral_constant<bool, is_actor<typename std::decay<L>::type>::value || is_actor<typename std::decay<R>::type>::value> {};

#define THRUST_CDNA4_PH_OPERATOR(SYM, OP)                                                                          \
  template <class L, class R, class = typename std::enable_if<either_is_actor<L, R>::value>::type>                  \
  THRUST_CDNA4_HD constexpr actor<binary_expr<OP, typename as_node<L>::type, typename as_node<R>::type>> operator SYM(const L& l, const R& r) { \
    typedef binary_expr<OP, typename as_node<L>::type, typename as_node<R>::type> node;                             \
    return actor<node>(node{as_node<L>::make(l), as_node<R>::make(r)});                                            \
  }
THRUST_CDNA4_PH_OPERATOR(+, op_plus)
THRUST_CDNA4_PH_OPERATOR(-, op_minus)
THRUST_CDNA4_PH_OPERATOR(*, op_mul)
THRUST_CDNA4_PH_OPERATOR(/, op_div)
THRUST_CDNA4_PH_OPERATOR(%, op_mod)
THRUST_CDNA4_PH_OPERATOR(<, op_lt)
THRUST_CDNA4_PH_OPERATOR(>, op_gt)
THRUST_CDNA4_PH_OPERATOR(<=, op_le)
THRUST_CDNA4_PH_OPERATOR(>=, op_ge)
THRUST_CDNA4_PH_OPERATOR(==, op_eq)
THRUST_CDNA4_PH_OPERATOR(!=, op_ne)
THRUST_CDNA4_PH_OPERATOR(&&, op_and)
THRUST_CDNA4_PH_OPERATOR(||, op_or)
THRUST_CDNA4_PH_OPERATOR(&, op_bit_and)
THRUST_CDNA4_PH_OPERATOR(|, op_bit_or)
THRUST_CDNA4_PH_OPERATOR(^, op_bit_xor)
THRUST_CDNA4_PH_OPERATOR(<<, op_shl)
THRUST_CDNA4_PH_OPERATOR(>>, op_shr)
#undef THRUST_CDNA4_PH_OPERATOR
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_negate, E>> operator-(const actor<E>& e) { return actor<unary_expr<op_negate, E>>(unary_expr<op_negate, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_not, E>> operator!(const actor<E>& e) { return actor<unary_expr<op_not, E>>(unary_expr<op_not, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_bit_not, E>> operator~(const actor<E>& e) { return actor<unary_expr<op_bit_not, E>>(unary_expr<op_bit_not, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_unary_plus, E>> operator+(const actor<E>& e) { return actor<unary_expr<op_unary_plus, E>>(unary_expr<op_unary_plus, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_pre_inc, E>> operator++(const actor<E>& e) { return actor<unary_expr<op_pre_inc, E>>(unary_expr<op_pre_inc, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_pre_dec, E>> operator--(const actor<E>& e) { return actor<unary_expr<op_pre_dec, E>>(unary_expr<op_pre_dec, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_post_inc, E>> operator++(const actor<E>& e, int) { return actor<unary_expr<op_post_inc, E>>(unary_expr<op_post_inc, E>{e}); }
template <class E> THRUST_CDNA4_HD constexpr actor<unary_expr<op_post_dec, E>> operator--(const actor<E>& e, int) { return actor<unary_expr<op_post_dec, E>>(unary_expr<op_post_dec, E>{e}); }

}}  // namespace detail::functional

namespace placeholders {
#define THRUST_CDNA4_PLACEHOLDER(N, I) static constexpr thrust::detail::functional::actor<thrust::detail::functional::argument<I>> N{};
THRUST_CDNA4_PLACEHOLDER(_1, 0)
THRUST_CDNA4_PLACEHOLDER(_2, 1)
THRUST_CDNA4_PLACEHOLDER(_3, 2)
THRUST_CDNA4_PLACEHOLDER(_4, 3)
THRUST_CDNA4_PLACEHOLDER(_5, 4)
THRUST_CDNA4_PLACEHOLDER(_6, 5)
THRUST_CDNA4_PLACEHOLDER(_7, 6)
THRUST_CDNA4_PLACEHOLDER(_8, 7)
THRUST_CDNA4_PLACEHOLDER(_9, 8)
THRUST_CDNA4_PLACEHOLDER(_10, 9)
#undef THRUST_CDNA4_PLACEHOLDER
}  // namespace placeholders
}  // namespace thrust
