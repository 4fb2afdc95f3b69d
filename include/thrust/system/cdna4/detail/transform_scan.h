// The cdna4 device system adds nothing of its own here (the reference's device systems leave such
// files empty to inherit the generic algorithm, e.g. thrust/system/cuda/detail/temporary_buffer.h:17-22):
// transform_inclusive_scan / transform_exclusive_scan are a scan over a transform_iterator.
#pragma once
#include <thrust/transform_scan.h>
