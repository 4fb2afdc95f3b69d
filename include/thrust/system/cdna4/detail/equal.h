// The cdna4 device system adds nothing of its own here (the reference's device systems leave such
// files empty to inherit the generic algorithm, e.g. thrust/system/cuda/detail/temporary_buffer.h:17-22):
// equal is a mismatch.
#pragma once
#include <thrust/equal.h>
