// <thrust/detail/cpp11_required.h>: every compiler these headers build with is C++14 or later.
#pragma once
#include <thrust/detail/config.h>
