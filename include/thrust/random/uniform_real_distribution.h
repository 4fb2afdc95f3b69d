// <thrust/random/uniform_real_distribution.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
