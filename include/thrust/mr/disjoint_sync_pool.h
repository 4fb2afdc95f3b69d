// thrust::mr::disjoint_synchronized_pool_resource (thrust/mr/disjoint_sync_pool.h): the disjoint
// caching pool behind a mutex.
#pragma once
#include <mutex>
#include <thrust/mr/disjoint_pool.h>
namespace thrust { namespace mr {
template <class Upstream, class Bookkeeper>
class disjoint_synchronized_pool_resource : public memory_resource<typename Upstream::pointer> {
  typedef disjoint_unsynchronized_pool_resource<Upstream, Bookkeeper> unsync_pool;
 public:
  typedef typename Upstream::pointer pointer;
  static pool_options get_default_options() { return unsync_pool::get_default_options(); }
  disjoint_synchronized_pool_resource(Upstream* upstream, Bookkeeper* bookkeeper, pool_options options = get_default_options())
      : pool_(upstream, bookkeeper, options) {}
  explicit disjoint_synchronized_pool_resource(pool_options options = get_default_options()) : pool_(options) {}
  void release() {
    std::lock_guard<std::mutex> lock(mutex_);
    pool_.release();
  }
  pointer do_allocate(std::size_t bytes, std::size_t alignment) override {
    std::lock_guard<std::mutex> lock(mutex_);
    return pool_.do_allocate(bytes, alignment);
  }
  void do_deallocate(pointer p, std::size_t bytes, std::size_t alignment) override {
    std::lock_guard<std::mutex> lock(mutex_);
    pool_.do_deallocate(p, bytes, alignment);
  }
 private:
  std::mutex mutex_;
  unsync_pool pool_;
};
}}  // namespace thrust::mr
