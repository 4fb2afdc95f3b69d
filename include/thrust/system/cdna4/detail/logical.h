// The cdna4 device system adds nothing of its own here (the reference's device systems leave such
// files empty to inherit the generic algorithm, e.g. thrust/system/cuda/detail/temporary_buffer.h:17-22):
// all_of / any_of / none_of are a find_if.
#pragma once
#include <thrust/logical.h>
