// thrust::conjunction / disjunction / negation and their _value forms
// (thrust/type_traits/logical_metafunctions.h).
#pragma once
#include <type_traits>
namespace thrust {
template <class... Ts> struct conjunction : std::true_type {};
template <class T> struct conjunction<T> : T {};
template <class T, class... Ts> struct conjunction<T, Ts...> : std::conditional<bool(T::value), conjunction<Ts...>, T>::type {};
template <class... Ts> struct disjunction : std::false_type {};
template <class T> struct disjunction<T> : T {};
template <class T, class... Ts> struct disjunction<T, Ts...> : std::conditional<bool(T::value), T, disjunction<Ts...>>::type {};
template <class T> struct negation : std::integral_constant<bool, !bool(T::value)> {};
// the same over plain bool values
template <bool... Bs> struct conjunction_value;
template <> struct conjunction_value<> : std::true_type {};
template <bool B, bool... Bs> struct conjunction_value<B, Bs...> : std::integral_constant<bool, B && conjunction_value<Bs...>::value> {};
template <bool... Bs> struct disjunction_value;
template <> struct disjunction_value<> : std::false_type {};
template <bool B, bool... Bs> struct disjunction_value<B, Bs...> : std::integral_constant<bool, B || disjunction_value<Bs...>::value> {};
template <bool B> struct negation_value : std::integral_constant<bool, !B> {};
#if __cplusplus >= 201402L
template <class... Ts> constexpr bool conjunction_v = conjunction<Ts...>::value;
template <class... Ts> constexpr bool disjunction_v = disjunction<Ts...>::value;
template <class T> constexpr bool negation_v = negation<T>::value;
template <bool... Bs> constexpr bool conjunction_value_v = conjunction_value<Bs...>::value;
template <bool... Bs> constexpr bool disjunction_value_v = disjunction_value<Bs...>::value;
template <bool B> constexpr bool negation_value_v = negation_value<B>::value;
#endif
}  // namespace thrust
