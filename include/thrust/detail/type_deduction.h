// <thrust/detail/type_deduction.h>: THRUST_FWD, THRUST_MVCAP, THRUST_RETURNS, THRUST_DECLTYPE_RETURNS.
#pragma once
#include <thrust/detail/config.h>
