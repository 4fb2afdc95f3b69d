// thrust::device_free (thrust/device_free.h): defined with device_ptr.
#pragma once
#include <thrust/device_ptr.h>
