// thrust::mr::disjoint_unsynchronized_pool_resource (thrust/mr/disjoint_pool.h): the caching pool
// of <thrust/mr/pool.h> with its records (free lists, chunk table) kept in memory of a second
// resource, the bookkeeper.  The pooled memory itself is never read or written by the pool, so it
// may be memory the host cannot address; the bookkeeper's memory must be host-addressable.
#pragma once
#include <thrust/mr/allocator.h>
#include <thrust/mr/pool.h>
namespace thrust { namespace mr {
namespace detail {
template <class Bookkeeper> struct resource_bookkeeping {
  Bookkeeper* resource;
  template <class T> struct alloc { typedef mr::allocator<T, Bookkeeper> type; };
  template <class T> mr::allocator<T, Bookkeeper> get() const { return mr::allocator<T, Bookkeeper>(resource); }
};
}  // namespace detail
template <class Upstream, class Bookkeeper>
class disjoint_unsynchronized_pool_resource final : public detail::pool_core<Upstream, detail::resource_bookkeeping<Bookkeeper>> {
  typedef detail::pool_core<Upstream, detail::resource_bookkeeping<Bookkeeper>> core;
 public:
  static pool_options get_default_options() { return detail::default_pool_options(); }
  disjoint_unsynchronized_pool_resource(Upstream* upstream, Bookkeeper* bookkeeper, pool_options options = get_default_options())
      : core(upstream, detail::resource_bookkeeping<Bookkeeper>{bookkeeper}, options) {}
  explicit disjoint_unsynchronized_pool_resource(pool_options options = get_default_options())
      : core(get_global_resource<Upstream>(), detail::resource_bookkeeping<Bookkeeper>{get_global_resource<Bookkeeper>()}, options) {}
};
}}  // namespace thrust::mr
