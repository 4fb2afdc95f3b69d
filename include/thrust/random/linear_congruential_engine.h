// <thrust/random/linear_congruential_engine.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
