// The cdna4 device system's per-device resources (the counterpart of
// thrust/system/cuda/detail/per_device_resource.h): one instance per device, keyed by the device that
// is current; thrust::get_per_device_resource in <thrust/per_device_resource.h> holds the table.
#pragma once
#include <thrust/per_device_resource.h>
