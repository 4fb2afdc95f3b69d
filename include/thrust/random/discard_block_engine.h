// <thrust/random/discard_block_engine.h>: defined in <thrust/random.h>.
#pragma once
#include <thrust/random.h>
