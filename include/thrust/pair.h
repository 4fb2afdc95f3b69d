// thrust::pair / make_pair / get / tuple_element / tuple_size (thrust/pair.h): a pair whose members
// are callable on the device (std::pair's assignment is not, before C++20), convertible from and
// to std::pair.
#pragma once
#include <cstddef>
#include <type_traits>
#include <utility>
#include <thrust/detail/hd.h>
#include <thrust/detail/swap.h>

namespace thrust {
template <class T1, class T2>
struct pair {
  typedef T1 first_type;
  typedef T2 second_type;
  T1 first;
  T2 second;

  // the members are value-initialised (thrust/pair.h:82-85; testing/pair.cu:13-16)
  THRUST_CDNA4_HD constexpr pair() : first(), second() {}
  THRUST_CDNA4_HD constexpr pair(const T1& x, const T2& y) : first(x), second(y) {}
  template <class U1, class U2, class = typename std::enable_if<std::is_convertible<const U1&, T1>::value && std::is_convertible<const U2&, T2>::value>::type>
  THRUST_CDNA4_HD constexpr pair(const pair<U1, U2>& p) : first(p.first), second(p.second) {}
  template <class U1, class U2, class = typename std::enable_if<std::is_convertible<const U1&, T1>::value && std::is_convertible<const U2&, T2>::value>::type>
  constexpr pair(const std::pair<U1, U2>& p) : first(p.first), second(p.second) {}
  pair(const pair&) = default;
  pair& operator=(const pair&) = default;
  template <class U1, class U2>
  THRUST_CDNA4_HD pair& operator=(const pair<U1, U2>& p) {
    first = p.first;
    second = p.second;
    return *this;
  }
  template <class U1, class U2> operator std::pair<U1, U2>() const { return std::pair<U1, U2>(first, second); }
  // member by member, each with the swap its type provides (thrust/pair.h: pair::swap)
  THRUST_CDNA4_HD void swap(pair& p) {
    detail::adl_swap(first, p.first);
    detail::adl_swap(second, p.second);
  }
};
template <class T1, class T2>
THRUST_CDNA4_HD inline void swap(pair<T1, T2>& x, pair<T1, T2>& y) { x.swap(y); }

template <class T1, class T2>
THRUST_CDNA4_HD constexpr pair<typename std::decay<T1>::type, typename std::decay<T2>::type> make_pair(T1&& x, T2&& y) {
  return pair<typename std::decay<T1>::type, typename std::decay<T2>::type>(static_cast<T1&&>(x), static_cast<T2&&>(y));
}
template <class T1, class T2> THRUST_CDNA4_HD constexpr bool operator==(const pair<T1, T2>& x, const pair<T1, T2>& y) { return x.first == y.first && x.second == y.second; }
template <class T1, class T2> THRUST_CDNA4_HD constexpr bool operator!=(const pair<T1, T2>& x, const pair<T1, T2>& y) { return !(x == y); }
template <class T1, class T2> THRUST_CDNA4_HD constexpr bool operator<(const pair<T1, T2>& x, const pair<T1, T2>& y) {
  return x.first < y.first || (!(y.first < x.first) && x.second < y.second);
}
template <class T1, class T2> THRUST_CDNA4_HD constexpr bool operator>(const pair<T1, T2>& x, const pair<T1, T2>& y) { return y < x; }
template <class T1, class T2> THRUST_CDNA4_HD constexpr bool operator<=(const pair<T1, T2>& x, const pair<T1, T2>& y) { return !(y < x); }
template <class T1, class T2> THRUST_CDNA4_HD constexpr bool operator>=(const pair<T1, T2>& x, const pair<T1, T2>& y) { return !(x < y); }

template <std::size_t I, class T> struct tuple_element;
template <class T> struct tuple_size;
template <class T1, class T2> struct tuple_element<0, pair<T1, T2>> { typedef T1 type; };
template <class T1, class T2> struct tuple_element<1, pair<T1, T2>> { typedef T2 type; };
template <class T1, class T2> struct tuple_size<pair<T1, T2>> : std::integral_constant<std::size_t, 2> {};
namespace detail {
template <std::size_t I> struct pair_get;
template <> struct pair_get<0> {
  template <class P> THRUST_CDNA4_HD static constexpr auto get(P& p) -> decltype((p.first)) { return p.first; }
};
template <> struct pair_get<1> {
  template <class P> THRUST_CDNA4_HD static constexpr auto get(P& p) -> decltype((p.second)) { return p.second; }
};
}  // namespace detail
template <std::size_t I, class T1, class T2>
THRUST_CDNA4_HD constexpr typename tuple_element<I, pair<T1, T2>>::type& get(pair<T1, T2>& p) { return detail::pair_get<I>::get(p); }
template <std::size_t I, class T1, class T2>
THRUST_CDNA4_HD constexpr const typename tuple_element<I, pair<T1, T2>>::type& get(const pair<T1, T2>& p) { return detail::pair_get<I>::get(p); }
}  // namespace thrust
