// thrust::integer_sequence, index_sequence, the make_ forms, the reversed forms and push_front /
// push_back (thrust/type_traits/integer_sequence.h).
#pragma once
#include <cstddef>
#include <utility>
namespace thrust {
template <class T, T... Is> using integer_sequence = std::integer_sequence<T, Is...>;
template <std::size_t... Is> using index_sequence = std::index_sequence<Is...>;
template <class T, std::size_t N> using make_integer_sequence = std::make_integer_sequence<T, N>;
template <std::size_t N> using make_index_sequence = std::make_index_sequence<N>;
namespace detail {
template <class T, T Value, class Sequence> struct integer_sequence_push_front_impl;
template <class T, T Value, T... Is> struct integer_sequence_push_front_impl<T, Value, integer_sequence<T, Is...>> {
  typedef integer_sequence<T, Value, Is...> type;
};
template <class T, T Value, class Sequence> struct integer_sequence_push_back_impl;
template <class T, T Value, T... Is> struct integer_sequence_push_back_impl<T, Value, integer_sequence<T, Is...>> {
  typedef integer_sequence<T, Is..., Value> type;
};
template <class T, std::size_t N> struct make_reversed_integer_sequence_impl {
  typedef typename integer_sequence_push_front_impl<T, (T)(N - 1), typename make_reversed_integer_sequence_impl<T, N - 1>::type>::type type;
};
template <class T> struct make_reversed_integer_sequence_impl<T, 0> { typedef integer_sequence<T> type; };
}  // namespace detail
template <class T, T Value, class Sequence> using integer_sequence_push_front = typename detail::integer_sequence_push_front_impl<T, Value, Sequence>::type;
template <class T, T Value, class Sequence> using integer_sequence_push_back = typename detail::integer_sequence_push_back_impl<T, Value, Sequence>::type;
template <class T, std::size_t N> using make_reversed_integer_sequence = typename detail::make_reversed_integer_sequence_impl<T, N>::type;
template <std::size_t N> using make_reversed_index_sequence = make_reversed_integer_sequence<std::size_t, N>;
}  // namespace thrust
