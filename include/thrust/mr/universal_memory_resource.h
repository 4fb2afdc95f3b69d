// thrust/mr/universal_memory_resource.h: thrust::universal_memory_resource and
// thrust::universal_host_pinned_memory_resource are the cdna4 system's.
#pragma once
#include <thrust/system/cdna4/memory_resource.h>
