// <thrust/detail/static_assert.h>: THRUST_STATIC_ASSERT and the dependent-false helpers
// (thrust/detail/static_assert.h:30-92).
#pragma once
#include <thrust/detail/config.h>
#include <type_traits>
#include <thrust/detail/preprocessor.h>
#define THRUST_STATIC_ASSERT(B) static_assert(B, "static assertion failed")
#define THRUST_STATIC_ASSERT_MSG(B, msg) static_assert(B, msg)
namespace thrust { namespace detail {
// false whatever T is, but only known once T is: for static_asserts in templates that must not
// fire before instantiation
template <class T, bool x> struct depend_on_instantiation { static constexpr bool value = x; };
}}  // namespace thrust::detail
