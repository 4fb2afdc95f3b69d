// <thrust/random/uniform_int_distribution.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
