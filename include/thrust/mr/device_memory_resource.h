// thrust/mr/device_memory_resource.h: thrust::device_memory_resource is the cdna4 system's.
#pragma once
#include <thrust/system/cdna4/memory_resource.h>
