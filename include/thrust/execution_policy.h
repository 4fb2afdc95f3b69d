// thrust::device, thrust::host and the cdna4 stream policies (thrust/execution_policy.h:295, :344).
#pragma once
#include <thrust/system/cdna4/detail/core.h>
