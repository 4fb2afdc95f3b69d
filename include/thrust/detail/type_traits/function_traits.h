// <thrust/detail/type_traits/function_traits.h>: is_adaptable_*_function, is_commutative.
#pragma once
#include <thrust/detail/type_traits.h>
#include <thrust/functional.h>
