// The cdna4 device system adds nothing of its own here (the reference's device systems leave such
// files empty to inherit the generic algorithm, e.g. thrust/system/cuda/detail/temporary_buffer.h:17-22):
// lower_bound / upper_bound / binary_search / equal_range run the system's search kernels (scalar_search, vector_search), which take the policy for its stream.
#pragma once
#include <thrust/binary_search.h>
