// The cdna4 device system adds nothing of its own here (the reference's device systems leave such
// files empty to inherit the generic algorithm, e.g. thrust/system/cuda/detail/temporary_buffer.h:17-22):
// unique_by_key and unique_by_key_copy live with unique in detail/unique.h.
#pragma once
#include <thrust/unique.h>
