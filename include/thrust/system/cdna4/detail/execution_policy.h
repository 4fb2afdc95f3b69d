// thrust::system::cdna4::tag and execution_policy<Derived> (the counterpart of
// thrust/system/cuda/detail/execution_policy.h:48-71).  Both are defined with the system's core
// (error category, policies, temporary storage) in core.h; this header is the name the reference's
// layout gives them.
#pragma once
#include <thrust/system/cdna4/detail/core.h>
