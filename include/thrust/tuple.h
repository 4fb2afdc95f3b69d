// thrust::tuple / get / make_tuple / tie / tuple_element / tuple_size (thrust/tuple.h): a small
// tuple whose members are callable on the device (std::tuple's assignment is not, before C++20),
// with element-wise conversion and assignment so that a tuple of references — what a
// zip_iterator dereferences to — reads from and writes to a tuple of values.
#pragma once
#include <cstddef>
#include <type_traits>
#include <utility>
#include <thrust/detail/hd.h>
#include <thrust/detail/swap.h>

namespace thrust {
template <class... Ts> struct tuple;
template <class T1, class T2> struct pair;
// the type the reference's ten-parameter tuple pads itself with (thrust/tuple.h:50); this tuple is
// variadic and has no use for it beyond existing code that names it
struct null_type {};

namespace detail {
template <std::size_t I, class T> struct tuple_leaf {
  T value;
};
// a reference member assigns through (and keeps tuples of values trivially copyable)
template <std::size_t I, class T> struct tuple_leaf<I, T&> {
  T& value;
  THRUST_CDNA4_HD tuple_leaf& operator=(const tuple_leaf& o) {
    value = o.value;
    return *this;
  }
};
template <std::size_t I, class... Ts> struct nth_type;
template <class T, class... Ts> struct nth_type<0, T, Ts...> { typedef T type; };
template <std::size_t I, class T, class... Ts> struct nth_type<I, T, Ts...> { typedef typename nth_type<I - 1, Ts...>::type type; };

template <class... Us> struct is_single_tuple : std::false_type {};
template <class... Ts> struct is_single_tuple<tuple<Ts...>> : std::true_type {};

template <class Seq, class... Ts> struct tuple_impl;
template <std::size_t... Is, class... Ts>
struct tuple_impl<std::index_sequence<Is...>, Ts...> : tuple_leaf<Is, Ts>... {
  tuple_impl() = default;
  THRUST_CDNA4_HD constexpr tuple_impl(const Ts&... vs) : tuple_leaf<Is, Ts>{vs}... {}
  template <class... Us>
  THRUST_CDNA4_HD constexpr tuple_impl(const tuple_impl<std::index_sequence<Is...>, Us...>& o)
      : tuple_leaf<Is, Ts>{static_cast<Ts>(static_cast<const tuple_leaf<Is, Us>&>(o).value)}... {}
  template <class... Us>
  THRUST_CDNA4_HD void assign(const tuple_impl<std::index_sequence<Is...>, Us...>& o) {
    int unused[] = {0, ((void)(static_cast<tuple_leaf<Is, Ts>&>(*this).value = static_cast<const tuple_leaf<Is, Us>&>(o).value), 0)...};
    (void)unused;
  }
  template <class... Us>
  THRUST_CDNA4_HD constexpr bool equals(const tuple_impl<std::index_sequence<Is...>, Us...>& o) const {
    bool same = true;
    int unused[] = {0, ((void)(same = same && (static_cast<const tuple_leaf<Is, Ts>&>(*this).value == static_cast<const tuple_leaf<Is, Us>&>(o).value)), 0)...};
    (void)unused;
    return same;
  }
};
}  // namespace detail

template <class... Ts>
struct tuple : detail::tuple_impl<std::index_sequence_for<Ts...>, Ts...> {
  typedef detail::tuple_impl<std::index_sequence_for<Ts...>, Ts...> base;
  tuple() = default;
  tuple(const tuple&) = default;
  template <class... Us, class = typename std::enable_if<sizeof...(Us) == sizeof...(Ts) && (sizeof...(Ts) > 0) &&
                                                         !detail::is_single_tuple<typename std::decay<Us>::type...>::value>::type>
  THRUST_CDNA4_HD constexpr tuple(Us&&... vs) : base(static_cast<Us&&>(vs)...) {}
  template <class... Us, class = typename std::enable_if<sizeof...(Us) == sizeof...(Ts)>::type>
  THRUST_CDNA4_HD constexpr tuple(const tuple<Us...>& o) : base(static_cast<const typename tuple<Us...>::base&>(o)) {}
  tuple& operator=(const tuple&) = default;
  template <class... Us>
  THRUST_CDNA4_HD tuple& operator=(const tuple<Us...>& o) {
    base::assign(static_cast<const typename tuple<Us...>::base&>(o));
    return *this;
  }
  // a tuple of two from and to a pair (thrust/tuple.h: tuple<T0, T1>::operator=(const pair<U1, U2>&))
  template <class U1, class U2, class = typename std::enable_if<sizeof...(Ts) == 2 && (sizeof(U1) > 0)>::type>
  THRUST_CDNA4_HD constexpr tuple(const pair<U1, U2>& p) : base(p.first, p.second) {}
  template <class U1, class U2>
  THRUST_CDNA4_HD tuple& operator=(const pair<U1, U2>& p) {
    static_cast<detail::tuple_leaf<0, typename detail::nth_type<0, Ts...>::type>&>(*this).value = p.first;
    static_cast<detail::tuple_leaf<1, typename detail::nth_type<1, Ts...>::type>&>(*this).value = p.second;
    return *this;
  }
  template <class U1, class U2>
  THRUST_CDNA4_HD const tuple& operator=(const pair<U1, U2>& p) const {
    *const_cast<tuple*>(this) = p;
    return *this;
  }
  // a tuple of references assigns through them, also when it is a temporary
  template <class... Us>
  THRUST_CDNA4_HD const tuple& operator=(const tuple<Us...>& o) const {
    const_cast<tuple*>(this)->base::assign(static_cast<const typename tuple<Us...>::base&>(o));
    return *this;
  }
};
template <> struct tuple<> {};

template <std::size_t I, class T> struct tuple_element;
template <std::size_t I, class... Ts> struct tuple_element<I, tuple<Ts...>> { typedef typename detail::nth_type<I, Ts...>::type type; };
template <std::size_t I, class T> struct tuple_element<I, const T> { typedef typename std::add_const<typename tuple_element<I, T>::type>::type type; };
template <std::size_t I, class T> struct tuple_element<I, volatile T> { typedef typename std::add_volatile<typename tuple_element<I, T>::type>::type type; };
template <std::size_t I, class T> struct tuple_element<I, const volatile T> { typedef typename std::add_cv<typename tuple_element<I, T>::type>::type type; };
template <class T> struct tuple_size;
// how an element of a tuple is handed out (thrust/tuple.h: access_traits, from the boost tuple)
template <class T> struct access_traits {
  typedef const T& const_type;
  typedef T& non_const_type;
  typedef const typename std::remove_cv<T>::type& parameter_type;
};
template <class T> struct access_traits<T&> {
  typedef T& const_type;
  typedef T& non_const_type;
  typedef T& parameter_type;
};
template <class... Ts> struct tuple_size<tuple<Ts...>> : std::integral_constant<std::size_t, sizeof...(Ts)> {};
template <class T> struct tuple_size<const T> : tuple_size<T> {};
template <class T> struct tuple_size<volatile T> : tuple_size<T> {};
template <class T> struct tuple_size<const volatile T> : tuple_size<T> {};

template <std::size_t I, class... Ts>
THRUST_CDNA4_HD constexpr typename detail::nth_type<I, Ts...>::type& get(tuple<Ts...>& t) {
  return static_cast<detail::tuple_leaf<I, typename detail::nth_type<I, Ts...>::type>&>(t).value;
}
template <std::size_t I, class... Ts>
THRUST_CDNA4_HD constexpr const typename detail::nth_type<I, Ts...>::type& get(const tuple<Ts...>& t) {
  return static_cast<const detail::tuple_leaf<I, typename detail::nth_type<I, Ts...>::type>&>(t).value;
}
template <class... Ts>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<Ts>::type...> make_tuple(const Ts&... vs) {
  return tuple<typename std::decay<Ts>::type...>(vs...);
}
template <class... Ts>
THRUST_CDNA4_HD constexpr tuple<Ts&...> tie(Ts&... vs) { return tuple<Ts&...>(vs...); }
// The same two for a fixed number of arguments (thrust/tuple.h:190-260 declares them that way).
// Called unqualified under `using namespace thrust` with arguments of std types — a host_vector's
// iterators —, std::make_tuple and std::tie are candidates too; a function template without a
// parameter pack is the more specialised one and is chosen.
template <class T0>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type> make_tuple(T0&& v0) {
  return tuple<typename std::decay<T0>::type>(static_cast<T0&&>(v0));
}
template <class T0, class T1>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type> make_tuple(T0&& v0, T1&& v1) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1));
}
template <class T0, class T1, class T2>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2));
}
template <class T0, class T1, class T2, class T3>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3));
}
template <class T0, class T1, class T2, class T3, class T4>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3, T4&& v4) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3), static_cast<T4&&>(v4));
}
template <class T0, class T1, class T2, class T3, class T4, class T5>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3, T4&& v4, T5&& v5) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3), static_cast<T4&&>(v4), static_cast<T5&&>(v5));
}
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3, T4&& v4, T5&& v5, T6&& v6) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3), static_cast<T4&&>(v4), static_cast<T5&&>(v5), static_cast<T6&&>(v6));
}
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6, class T7>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type, typename std::decay<T7>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3, T4&& v4, T5&& v5, T6&& v6, T7&& v7) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type, typename std::decay<T7>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3), static_cast<T4&&>(v4), static_cast<T5&&>(v5), static_cast<T6&&>(v6), static_cast<T7&&>(v7));
}
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6, class T7, class T8>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type, typename std::decay<T7>::type, typename std::decay<T8>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3, T4&& v4, T5&& v5, T6&& v6, T7&& v7, T8&& v8) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type, typename std::decay<T7>::type, typename std::decay<T8>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3), static_cast<T4&&>(v4), static_cast<T5&&>(v5), static_cast<T6&&>(v6), static_cast<T7&&>(v7), static_cast<T8&&>(v8));
}
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6, class T7, class T8, class T9>
THRUST_CDNA4_HD constexpr tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type, typename std::decay<T7>::type, typename std::decay<T8>::type, typename std::decay<T9>::type> make_tuple(T0&& v0, T1&& v1, T2&& v2, T3&& v3, T4&& v4, T5&& v5, T6&& v6, T7&& v7, T8&& v8, T9&& v9) {
  return tuple<typename std::decay<T0>::type, typename std::decay<T1>::type, typename std::decay<T2>::type, typename std::decay<T3>::type, typename std::decay<T4>::type, typename std::decay<T5>::type, typename std::decay<T6>::type, typename std::decay<T7>::type, typename std::decay<T8>::type, typename std::decay<T9>::type>(static_cast<T0&&>(v0), static_cast<T1&&>(v1), static_cast<T2&&>(v2), static_cast<T3&&>(v3), static_cast<T4&&>(v4), static_cast<T5&&>(v5), static_cast<T6&&>(v6), static_cast<T7&&>(v7), static_cast<T8&&>(v8), static_cast<T9&&>(v9));
}
template <class T0>
THRUST_CDNA4_HD constexpr tuple<T0&> tie(T0& v0) { return tuple<T0&>(v0); }
template <class T0, class T1>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&> tie(T0& v0, T1& v1) { return tuple<T0&, T1&>(v0, v1); }
template <class T0, class T1, class T2>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&> tie(T0& v0, T1& v1, T2& v2) { return tuple<T0&, T1&, T2&>(v0, v1, v2); }
template <class T0, class T1, class T2, class T3>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&> tie(T0& v0, T1& v1, T2& v2, T3& v3) { return tuple<T0&, T1&, T2&, T3&>(v0, v1, v2, v3); }
template <class T0, class T1, class T2, class T3, class T4>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&, T4&> tie(T0& v0, T1& v1, T2& v2, T3& v3, T4& v4) { return tuple<T0&, T1&, T2&, T3&, T4&>(v0, v1, v2, v3, v4); }
template <class T0, class T1, class T2, class T3, class T4, class T5>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&, T4&, T5&> tie(T0& v0, T1& v1, T2& v2, T3& v3, T4& v4, T5& v5) { return tuple<T0&, T1&, T2&, T3&, T4&, T5&>(v0, v1, v2, v3, v4, v5); }
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&> tie(T0& v0, T1& v1, T2& v2, T3& v3, T4& v4, T5& v5, T6& v6) { return tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&>(v0, v1, v2, v3, v4, v5, v6); }
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6, class T7>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&, T7&> tie(T0& v0, T1& v1, T2& v2, T3& v3, T4& v4, T5& v5, T6& v6, T7& v7) { return tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&, T7&>(v0, v1, v2, v3, v4, v5, v6, v7); }
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6, class T7, class T8>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&, T7&, T8&> tie(T0& v0, T1& v1, T2& v2, T3& v3, T4& v4, T5& v5, T6& v6, T7& v7, T8& v8) { return tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&, T7&, T8&>(v0, v1, v2, v3, v4, v5, v6, v7, v8); }
template <class T0, class T1, class T2, class T3, class T4, class T5, class T6, class T7, class T8, class T9>
THRUST_CDNA4_HD constexpr tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&, T7&, T8&, T9&> tie(T0& v0, T1& v1, T2& v2, T3& v3, T4& v4, T5& v5, T6& v6, T7& v7, T8& v8, T9& v9) { return tuple<T0&, T1&, T2&, T3&, T4&, T5&, T6&, T7&, T8&, T9&>(v0, v1, v2, v3, v4, v5, v6, v7, v8, v9); }

// swap: element by element; tuples of references (what a zip_iterator yields) are taken by value
// and swap what they refer to
namespace detail {
template <std::size_t I, std::size_t N> struct tuple_swap {
  template <class A, class B> THRUST_CDNA4_HD static void run(A& a, B& b) {
    adl_swap(get<I>(a), get<I>(b));
    tuple_swap<I + 1, N>::run(a, b);
  }
};
template <std::size_t N> struct tuple_swap<N, N> {
  template <class A, class B> THRUST_CDNA4_HD static void run(A&, B&) {}
};
}  // namespace detail
template <class... Ts>
THRUST_CDNA4_HD void swap(tuple<Ts...>& a, tuple<Ts...>& b) { detail::tuple_swap<0, sizeof...(Ts)>::run(a, b); }
template <class... Ts>
THRUST_CDNA4_HD void swap(tuple<Ts&...>&& a, tuple<Ts&...>&& b) { detail::tuple_swap<0, sizeof...(Ts)>::run(a, b); }

template <class... Ts, class... Us>
THRUST_CDNA4_HD constexpr bool operator==(const tuple<Ts...>& a, const tuple<Us...>& b) {
  return a.equals(static_cast<const typename tuple<Us...>::base&>(b));
}
template <class... Ts, class... Us>
THRUST_CDNA4_HD constexpr bool operator!=(const tuple<Ts...>& a, const tuple<Us...>& b) { return !(a == b); }

namespace detail {
template <std::size_t I, std::size_t N> struct tuple_less {
  template <class A, class B> THRUST_CDNA4_HD static constexpr bool run(const A& a, const B& b) {
    return get<I>(a) < get<I>(b) ? true : get<I>(b) < get<I>(a) ? false : tuple_less<I + 1, N>::run(a, b);
  }
};
template <std::size_t N> struct tuple_less<N, N> {
  template <class A, class B> THRUST_CDNA4_HD static constexpr bool run(const A&, const B&) { return false; }
};
}  // namespace detail
template <class... Ts, class... Us>
THRUST_CDNA4_HD constexpr bool operator<(const tuple<Ts...>& a, const tuple<Us...>& b) {
  return detail::tuple_less<0, sizeof...(Ts)>::run(a, b);
}
template <class... Ts, class... Us>
THRUST_CDNA4_HD constexpr bool operator>(const tuple<Ts...>& a, const tuple<Us...>& b) { return b < a; }
template <class... Ts, class... Us>
THRUST_CDNA4_HD constexpr bool operator<=(const tuple<Ts...>& a, const tuple<Us...>& b) { return !(b < a); }
template <class... Ts, class... Us>
THRUST_CDNA4_HD constexpr bool operator>=(const tuple<Ts...>& a, const tuple<Us...>& b) { return !(a < b); }
}  // namespace thrust
