// <thrust/random/xor_combine_engine.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
