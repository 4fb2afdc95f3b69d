// thrust::universal_ptr (thrust/universal_ptr.h): defined with universal_allocator.
#pragma once
#include <thrust/universal_allocator.h>
