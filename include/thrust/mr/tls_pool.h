// thrust::mr::tls_pool (thrust/mr/tls_pool.h): one unsynchronized caching pool per thread and
// upstream type.  The first call on a thread names the upstream; later calls may leave it out.
#pragma once
#include <cassert>
#include <thrust/mr/pool.h>
namespace thrust { namespace mr {
template <class Upstream>
unsynchronized_pool_resource<Upstream>& tls_pool(Upstream* upstream = nullptr) {
  static thread_local unsynchronized_pool_resource<Upstream> pool([&] {
    assert(upstream);
    return upstream;
  }());
  return pool;
}
}}  // namespace thrust::mr
