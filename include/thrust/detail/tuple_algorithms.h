// <thrust/detail/tuple_algorithms.h>: tuple_for_each, tuple_transform and tuple_subset over
// std::tuple (thrust/detail/tuple_algorithms.h:30-110).
#pragma once
#include <cstddef>
#include <tuple>
#include <type_traits>
#include <utility>
#include <thrust/detail/config.h>
#include <thrust/type_traits/integer_sequence.h>
namespace thrust {
namespace detail {
template <class Tuple, class F, std::size_t... Is>
auto tuple_transform_impl(Tuple&& t, F&& f, index_sequence<Is...>) -> decltype(std::make_tuple(f(std::get<Is>(std::forward<Tuple>(t)))...)) {
  return std::make_tuple(f(std::get<Is>(std::forward<Tuple>(t)))...);
}
template <class Tuple, class F, std::size_t... Is>
void tuple_for_each_impl(Tuple&& t, F&& f, index_sequence<Is...>) {
  int unused[] = {0, ((void)f(std::get<Is>(std::forward<Tuple>(t))), 0)...};
  (void)unused;
}
}  // namespace detail
// a tuple of f(element) for every element
template <class Tuple, class F>
auto tuple_transform(Tuple&& t, F&& f)
    -> decltype(detail::tuple_transform_impl(std::forward<Tuple>(t), std::forward<F>(f), make_index_sequence<std::tuple_size<typename std::decay<Tuple>::type>::value>{})) {
  return detail::tuple_transform_impl(std::forward<Tuple>(t), std::forward<F>(f), make_index_sequence<std::tuple_size<typename std::decay<Tuple>::type>::value>{});
}
// f(element) for every element, in order; returns the functor
template <class Tuple, class F>
typename std::decay<F>::type tuple_for_each(Tuple&& t, F&& f) {
  detail::tuple_for_each_impl(std::forward<Tuple>(t), f, make_index_sequence<std::tuple_size<typename std::decay<Tuple>::type>::value>{});
  return std::forward<F>(f);
}
// the elements at the given positions, in that order
template <class Tuple, std::size_t... Is>
auto tuple_subset(Tuple&& t, index_sequence<Is...>) -> decltype(std::make_tuple(std::get<Is>(std::forward<Tuple>(t))...)) {
  return std::make_tuple(std::get<Is>(std::forward<Tuple>(t))...);
}
}  // namespace thrust
