// thrust::mr::disjoint_tls_pool (thrust/mr/disjoint_tls_pool.h): one disjoint unsynchronized
// caching pool per thread and (upstream, bookkeeper) type pair.  The first call on a thread names
// both resources; later calls may leave them out.
#pragma once
#include <cassert>
#include <thrust/mr/disjoint_pool.h>
namespace thrust { namespace mr {
template <class Upstream, class Bookkeeper>
disjoint_unsynchronized_pool_resource<Upstream, Bookkeeper>& disjoint_tls_pool(Upstream* upstream = nullptr, Bookkeeper* bookkeeper = nullptr) {
  static thread_local disjoint_unsynchronized_pool_resource<Upstream, Bookkeeper> pool(
      [&] { assert(upstream); return upstream; }(), [&] { assert(bookkeeper); return bookkeeper; }());
  return pool;
}
}}  // namespace thrust::mr
