// <thrust/detail/type_traits.h>: the pre-C++11 style trait names that code written against Thrust's
// internals still spells thrust::detail::X — each one is the standard trait of the same meaning
// (thrust/detail/type_traits.h:36-560; is_commutative from
// thrust/detail/type_traits/function_traits.h:78-92).
#pragma once
#include <thrust/detail/config.h>
#include <type_traits>
#include <thrust/detail/cstdint.h>

namespace thrust {
template <class T> class device_reference;
template <class T> class device_ptr;
template <class T> struct plus;
template <class T> struct multiplies;
template <class T> struct minimum;
template <class T> struct maximum;
template <class T> struct logical_or;
template <class T> struct logical_and;
template <class T> struct bit_or;
template <class T> struct bit_and;
template <class T> struct bit_xor;

// thrust::integral_constant, true_type, false_type (thrust/detail/type_traits.h:37-63): the standard ones
using std::integral_constant;
using std::true_type;
using std::false_type;

namespace detail {
using std::integral_constant;
using std::true_type;
using std::false_type;
using std::conditional;
using std::enable_if;
using std::is_convertible;
using std::is_same;
using std::is_void;
using std::is_pointer;
using std::is_const;
using std::is_volatile;
using std::is_reference;
using std::is_floating_point;
using std::add_const;
using std::add_volatile;
using std::add_cv;
using std::remove_const;
using std::remove_volatile;
using std::remove_cv;
using std::remove_reference;
using std::is_base_of;
using std::make_unsigned;

template <class T> struct is_integral : std::is_integral<T> {};
template <class T> struct is_arithmetic : std::is_arithmetic<T> {};
template <class T> struct is_non_bool_integral : std::integral_constant<bool, std::is_integral<T>::value && !std::is_same<typename std::remove_cv<T>::type, bool>::value> {};
template <class T> struct is_non_bool_arithmetic : std::integral_constant<bool, std::is_arithmetic<T>::value && !std::is_same<typename std::remove_cv<T>::type, bool>::value> {};
template <class T> struct is_numeric : std::integral_constant<bool, std::is_convertible<int, T>::value && std::is_convertible<T, int>::value> {};
template <class T> struct is_pod : std::integral_constant<bool, std::is_void<T>::value || std::is_pointer<T>::value || std::is_arithmetic<T>::value || __is_pod(T)> {};
template <class T> struct has_trivial_constructor : std::integral_constant<bool, is_pod<T>::value || std::is_trivially_default_constructible<T>::value> {};
template <class T> struct has_trivial_copy_constructor : std::integral_constant<bool, is_pod<T>::value || std::is_trivially_copy_constructible<T>::value> {};
template <class T> struct has_trivial_destructor : is_pod<T> {};
template <class T> struct has_trivial_assign : std::integral_constant<bool, is_pod<T>::value || std::is_trivially_copy_assignable<T>::value> {};

template <class T> struct is_device_ptr : std::false_type {};
template <class T> struct is_device_ptr<device_ptr<T>> : std::true_type {};
template <class T> struct is_proxy_reference : std::false_type {};
template <class T> struct is_device_reference : std::false_type {};
template <class T> struct is_device_reference<device_reference<T>> : std::true_type {};
template <class T> struct is_reference_to_const : std::false_type {};
template <class T> struct is_reference_to_const<const T&> : std::true_type {};
// a reference through which a functor's result can be stored (thrust/detail/type_traits.h: user
// code specialises it for proxy references of its own, testing/copy.cu:737-744)
template <class T> struct is_non_const_reference
    : std::integral_constant<bool, std::is_lvalue_reference<T>::value && !is_reference_to_const<T>::value> {};
template <class T> struct add_reference { typedef typename std::add_lvalue_reference<T>::type type; };

template <class A, class B> struct lazy_is_same : std::is_same<typename A::type, typename B::type> {};
template <class A, class B> struct is_different : std::integral_constant<bool, !std::is_same<A, B>::value> {};
template <class A, class B> struct lazy_is_different : is_different<typename A::type, typename B::type> {};
template <class A, class B> struct is_one_convertible_to_the_other : std::integral_constant<bool, std::is_convertible<A, B>::value || std::is_convertible<B, A>::value> {};

template <class... C> struct or_;
template <> struct or_<> : std::false_type {};
template <class C, class... R> struct or_<C, R...> : std::integral_constant<bool, C::value || or_<R...>::value> {};
template <class... C> struct and_;
template <> struct and_<> : std::true_type {};
template <class C, class... R> struct and_<C, R...> : std::integral_constant<bool, C::value && and_<R...>::value> {};
template <class C> struct not_ : std::integral_constant<bool, !C::value> {};

template <bool B, class Then, class Else> struct eval_if { typedef typename Then::type type; };
template <class Then, class Else> struct eval_if<false, Then, Else> { typedef typename Else::type type; };
template <class T> struct identity_ { typedef T type; };

template <bool B, class T> struct lazy_enable_if {};
template <class T> struct lazy_enable_if<true, T> { typedef typename T::type type; };
template <bool B, class T = void> struct disable_if : std::enable_if<!B, T> {};
template <bool B, class T> struct lazy_disable_if : lazy_enable_if<!B, T> {};
template <class A, class B, class T = void> struct enable_if_convertible : std::enable_if<std::is_convertible<A, B>::value, T> {};
template <class A, class B, class T = void> struct disable_if_convertible : std::enable_if<!std::is_convertible<A, B>::value, T> {};
template <class A, class B, class T = void> struct enable_if_different : std::enable_if<!std::is_same<A, B>::value, T> {};

struct largest_available_float { typedef double type; };
template <class A, class B> struct larger_type : std::conditional<(sizeof(B) > sizeof(A)), B, A> {};

template <class T> using invoke_result_unary_t = decltype(std::declval<T>()());

// has_result_type and friends (thrust/detail/type_traits/has_nested_type.h:22-42)
#define __THRUST_DEFINE_HAS_NESTED_TYPE(trait_name, nested_type_name)                            \
  template <class T_> struct trait_name {                                                        \
    template <class U_> static char (&test(typename U_::nested_type_name*))[1];                  \
    template <class U_> static char (&test(...))[2];                                             \
    static const bool value = sizeof(test<T_>(0)) == 1;                                          \
    typedef ::std::integral_constant<bool, value> type;                                          \
  };
__THRUST_DEFINE_HAS_NESTED_TYPE(has_result_type, result_type)
__THRUST_DEFINE_HAS_NESTED_TYPE(has_argument_type, argument_type)
__THRUST_DEFINE_HAS_NESTED_TYPE(has_first_argument_type, first_argument_type)
__THRUST_DEFINE_HAS_NESTED_TYPE(has_second_argument_type, second_argument_type)
template <class F> struct result_type { typedef typename F::result_type type; };
template <class F> struct is_adaptable_unary_function : std::integral_constant<bool, has_result_type<F>::value && has_argument_type<F>::value> {};
template <class F> struct is_adaptable_binary_function : std::integral_constant<bool, has_result_type<F>::value && has_first_argument_type<F>::value && has_second_argument_type<F>::value> {};

// which function objects may have their operands exchanged
template <class F> struct is_commutative : std::false_type {};
template <class T> struct is_commutative<plus<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<multiplies<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<minimum<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<maximum<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<logical_or<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<logical_and<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<bit_or<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<bit_and<T>> : std::is_arithmetic<T> {};
template <class T> struct is_commutative<bit_xor<T>> : std::is_arithmetic<T> {};
}  // namespace detail
}  // namespace thrust
