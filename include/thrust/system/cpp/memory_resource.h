// Memory resources of the host system (thrust/system/cpp/memory_resource.h): operator new / delete.
#pragma once
#include <thrust/mr/new.h>
namespace thrust { namespace system { namespace cpp {
typedef thrust::mr::new_delete_resource memory_resource;
typedef thrust::mr::new_delete_resource universal_memory_resource;
typedef thrust::mr::new_delete_resource universal_host_pinned_memory_resource;
}}}  // namespace thrust::system::cpp
