// <thrust/detail/type_traits/has_nested_type.h>: __THRUST_DEFINE_HAS_NESTED_TYPE.
#pragma once
#include <thrust/detail/type_traits.h>
