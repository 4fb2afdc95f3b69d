// thrust::system_error and the cdna4 error category (thrust/system/system_error.h,
// thrust/system/cuda/error.h).
#pragma once
#include <thrust/system/cdna4/detail/core.h>
