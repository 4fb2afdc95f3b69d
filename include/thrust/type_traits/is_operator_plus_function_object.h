// thrust::is_operator_plus_function_object (thrust/type_traits/is_operator_plus_function_object.h):
// whether a function object is known to be operator+ (thrust::plus, std::plus).
#pragma once
#include <functional>
#include <type_traits>
#include <thrust/functional.h>
namespace thrust {
namespace detail {
template <class F> struct is_operator_plus_function_object_impl : std::false_type {};
template <class T> struct is_operator_plus_function_object_impl<thrust::plus<T>> : std::true_type {};
template <class T> struct is_operator_plus_function_object_impl<std::plus<T>> : std::true_type {};
}  // namespace detail
template <class F> struct is_operator_plus_function_object : detail::is_operator_plus_function_object_impl<F> {};
#if __cplusplus >= 201402L
template <class F> constexpr bool is_operator_plus_function_object_v = is_operator_plus_function_object<F>::value;
#endif
}  // namespace thrust
