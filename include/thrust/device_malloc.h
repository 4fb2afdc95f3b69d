// thrust::device_malloc (thrust/device_malloc.h): defined with device_ptr.
#pragma once
#include <thrust/device_ptr.h>
