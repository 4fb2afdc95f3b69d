// thrust::is_trivially_relocatable, is_trivially_relocatable_to, is_indirectly_trivially_relocatable_to,
// proclaim_trivially_relocatable and THRUST_PROCLAIM_TRIVIALLY_RELOCATABLE
// (thrust/type_traits/is_trivially_relocatable.h): types whose objects may be moved with a plain
// byte copy (what a copy between host and device memory is).
#pragma once
#include <iterator>
#include <type_traits>
#include <thrust/type_traits/is_contiguous_iterator.h>
namespace thrust {
template <class T> struct proclaim_trivially_relocatable : std::false_type {};
#define THRUST_PROCLAIM_TRIVIALLY_RELOCATABLE(T) \
  namespace thrust { template <> struct proclaim_trivially_relocatable<T> : std::true_type {}; }
template <class T> struct is_trivially_relocatable
    : std::integral_constant<bool, std::is_trivially_copyable<T>::value || proclaim_trivially_relocatable<T>::value> {};
template <class From, class To> struct is_trivially_relocatable_to
    : std::integral_constant<bool, std::is_same<typename std::remove_cv<From>::type, typename std::remove_cv<To>::type>::value &&
                                       is_trivially_relocatable<typename std::remove_cv<To>::type>::value> {};
template <class FromIterator, class ToIterator> struct is_indirectly_trivially_relocatable_to
    : std::integral_constant<bool, is_contiguous_iterator<FromIterator>::value && is_contiguous_iterator<ToIterator>::value &&
                                       is_trivially_relocatable_to<typename std::iterator_traits<FromIterator>::value_type,
                                                                   typename std::iterator_traits<ToIterator>::value_type>::value> {};
#if __cplusplus >= 201402L
template <class T> constexpr bool is_trivially_relocatable_v = is_trivially_relocatable<T>::value;
template <class From, class To> constexpr bool is_trivially_relocatable_to_v = is_trivially_relocatable_to<From, To>::value;
template <class F, class T> constexpr bool is_indirectly_trivially_relocatable_to_v = is_indirectly_trivially_relocatable_to<F, T>::value;
#endif
}  // namespace thrust
