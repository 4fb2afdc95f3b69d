// The cdna4 device system adds nothing of its own here (the reference's device systems leave such
// files empty to inherit the generic algorithm, e.g. thrust/system/cuda/detail/temporary_buffer.h:17-22):
// the set operations are a per-element predicate on the select kernel plus a merge (set_operation).
#pragma once
#include <thrust/set_operations.h>
