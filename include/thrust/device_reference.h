// thrust::device_reference (thrust/device_reference.h): defined with device_ptr.
#pragma once
#include <thrust/device_ptr.h>
