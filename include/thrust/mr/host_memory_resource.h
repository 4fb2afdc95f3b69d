// thrust::host_memory_resource (thrust/mr/host_memory_resource.h): host memory from operator new.
#pragma once
#include <thrust/mr/new.h>
namespace thrust {
typedef mr::new_delete_resource host_memory_resource;
}  // namespace thrust
