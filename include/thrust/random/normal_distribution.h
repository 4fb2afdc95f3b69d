// <thrust/random/normal_distribution.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
