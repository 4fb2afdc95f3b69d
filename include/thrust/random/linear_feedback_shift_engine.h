// <thrust/random/linear_feedback_shift_engine.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
