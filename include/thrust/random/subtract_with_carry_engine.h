// <thrust/random/subtract_with_carry_engine.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
