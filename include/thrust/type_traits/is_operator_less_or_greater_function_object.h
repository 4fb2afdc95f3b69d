// thrust::is_operator_less_function_object / is_operator_greater_function_object /
// is_operator_less_or_greater_function_object
// (thrust/type_traits/is_operator_less_or_greater_function_object.h): whether a comparison object
// is known to be operator< or operator> — the test that sends a sort to the radix path
// (thrust/system/cuda/detail/sort.h:389-395).
#pragma once
#include <functional>
#include <type_traits>
#include <thrust/functional.h>
namespace thrust {
namespace detail {
template <class F> struct is_operator_less_function_object_impl : std::false_type {};
template <class T> struct is_operator_less_function_object_impl<thrust::less<T>> : std::true_type {};
template <class T> struct is_operator_less_function_object_impl<std::less<T>> : std::true_type {};
template <class F> struct is_operator_greater_function_object_impl : std::false_type {};
template <class T> struct is_operator_greater_function_object_impl<thrust::greater<T>> : std::true_type {};
template <class T> struct is_operator_greater_function_object_impl<std::greater<T>> : std::true_type {};
}  // namespace detail
template <class F> struct is_operator_less_function_object : detail::is_operator_less_function_object_impl<F> {};
template <class F> struct is_operator_greater_function_object : detail::is_operator_greater_function_object_impl<F> {};
template <class F> struct is_operator_less_or_greater_function_object
    : std::integral_constant<bool, is_operator_less_function_object<F>::value || is_operator_greater_function_object<F>::value> {};
#if __cplusplus >= 201402L
template <class F> constexpr bool is_operator_less_function_object_v = is_operator_less_function_object<F>::value;
template <class F> constexpr bool is_operator_greater_function_object_v = is_operator_greater_function_object<F>::value;
template <class F> constexpr bool is_operator_less_or_greater_function_object_v = is_operator_less_or_greater_function_object<F>::value;
#endif
}  // namespace thrust
