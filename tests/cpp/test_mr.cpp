// Memory resources, allocators and temporary storage from a user allocator, in the shape of
// the reference's testing/mr_new.cu, mr_pool.cu, mr_pool_options.cu, allocator.cu and
// examples/cuda/custom_temporary_allocation.cu.  Compiled by hipcc (thrust::reduce is a kernel template).
#include <map>

#include <thrust/device_allocator.h>
#include <thrust/device_vector.h>
#include <thrust/mr/allocator.h>
#include <thrust/mr/device_memory_resource.h>
#include <thrust/mr/disjoint_pool.h>
#include <thrust/mr/disjoint_sync_pool.h>
#include <thrust/mr/disjoint_tls_pool.h>
#include <thrust/mr/fancy_pointer_resource.h>
#include <thrust/mr/host_memory_resource.h>
#include <thrust/mr/new.h>
#include <thrust/mr/polymorphic_adaptor.h>
#include <thrust/mr/pool.h>
#include <thrust/mr/sync_pool.h>
#include <thrust/mr/tls_pool.h>
#include <thrust/mr/validator.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sort.h>

#include <thread>

#include "testing.h"

// counts what reaches it (testing/mr_pool.cu:30-80 uses a tracking upstream the same way)
template <class Upstream>
class tracking_resource final : public thrust::mr::memory_resource<typename Upstream::pointer> {
 public:
  typedef typename Upstream::pointer pointer;
  explicit tracking_resource(Upstream* up) : up_(up) {}
  pointer do_allocate(std::size_t bytes, std::size_t align) override {
    ++allocations; live_bytes += bytes;
    return up_->allocate(bytes, align);
  }
  void do_deallocate(pointer p, std::size_t bytes, std::size_t align) override {
    ++deallocations; live_bytes -= bytes;
    up_->deallocate(p, bytes, align);
  }
  int allocations = 0, deallocations = 0;
  std::size_t live_bytes = 0;
 private:
  Upstream* up_;
};

// testing/mr_new.cu:20-60
void TestNewDeleteResource() {
  thrust::mr::new_delete_resource r;
  void* p = r.allocate(100);
  ASSERT_TRUE(p != nullptr);
  static_cast<char*>(p)[99] = 1;
  r.deallocate(p, 100);
  void* q = r.allocate(64, 4096);
  ASSERT_EQUAL(reinterpret_cast<std::uintptr_t>(q) % 4096, (std::uintptr_t)0);
  r.deallocate(q, 64, 4096);
  thrust::mr::new_delete_resource other;
  ASSERT_TRUE(r == other);
}
DECLARE_UNITTEST(TestNewDeleteResource);

// testing/mr_pool.cu:120-260: caching, chunking, oversized blocks, release
template <class Upstream>
void pool_behaviour(Upstream* upstream) {
  tracking_resource<Upstream> tracker(upstream);
  {
    thrust::mr::pool_options opt = thrust::mr::unsynchronized_pool_resource<thrust::mr::new_delete_resource>::get_default_options();
    opt.smallest_block_size = 256;
    opt.largest_block_size = 1 << 16;
    opt.min_blocks_per_chunk = 4;
    opt.min_bytes_per_chunk = 1024;
    ASSERT_TRUE(opt.validate());
    thrust::mr::unsynchronized_pool_resource<tracking_resource<Upstream>> pool(&tracker, opt);
    auto a = pool.allocate(1000);  // class 1024: one chunk of 4 blocks
    ASSERT_EQUAL(tracker.allocations, 1);
    auto b = pool.allocate(1024);
    auto c = pool.allocate(600);
    auto d = pool.allocate(513);
    ASSERT_EQUAL(tracker.allocations, 1);
    ASSERT_TRUE(a != b && b != c && c != d && a != d);
    auto e = pool.allocate(1024);  // the chunk is used up: a second one
    ASSERT_EQUAL(tracker.allocations, 2);
    pool.deallocate(b, 1024);
    auto f = pool.allocate(700);  // comes back from the free list
    ASSERT_TRUE(f == b);
    ASSERT_EQUAL(tracker.allocations, 2);
    auto g = pool.allocate(100);  // another size class
    ASSERT_EQUAL(tracker.allocations, 3);
    // oversized: straight from the upstream, cached on deallocate
    auto big = pool.allocate(1 << 20);
    ASSERT_EQUAL(tracker.allocations, 4);
    pool.deallocate(big, 1 << 20);
    ASSERT_EQUAL(tracker.deallocations, 0);
    auto big2 = pool.allocate((1 << 20) - 4096);
    ASSERT_TRUE(big2 == big);
    ASSERT_EQUAL(tracker.allocations, 4);
    auto big3 = pool.allocate(1 << 17);  // too small for the cached block's cutoff? no: it is in use
    ASSERT_EQUAL(tracker.allocations, 5);
    pool.deallocate(big2, (1 << 20) - 4096);
    pool.deallocate(big3, 1 << 17);
    for (auto p : {a, c, d, e, f}) pool.deallocate(p, 1024);
    pool.deallocate(g, 100);
    ASSERT_EQUAL(tracker.deallocations, 0);  // nothing returns before release
    pool.release();
    ASSERT_EQUAL(tracker.deallocations, 5);
    ASSERT_EQUAL(tracker.live_bytes, (std::size_t)0);
    auto again = pool.allocate(1024);  // usable after release
    ASSERT_EQUAL(tracker.allocations, 6);
    pool.deallocate(again, 1024);
  }
  ASSERT_EQUAL(tracker.allocations, tracker.deallocations);  // the destructor releases
  thrust::mr::pool_options bad;
  bad.smallest_block_size = 3;
  ASSERT_TRUE(!bad.validate());
  ASSERT_THROWS(thrust::mr::unsynchronized_pool_resource<tracking_resource<Upstream>>(&tracker, bad), std::invalid_argument);
}
void TestPoolOverHostMemory() {
  thrust::mr::new_delete_resource up;
  pool_behaviour(&up);
}
DECLARE_UNITTEST(TestPoolOverHostMemory);
void TestPoolOverDeviceMemory() {
  thrust::device_memory_resource up;  // hipMalloc / hipFree
  pool_behaviour(&up);
}
DECLARE_UNITTEST(TestPoolOverDeviceMemory);

// testing/allocator.cu:60-140: a device_vector over a user pool, allocator equality and rebind
void TestDeviceVectorWithPoolAllocator() {
  typedef thrust::mr::unsynchronized_pool_resource<thrust::device_memory_resource> Pool;
  typedef thrust::mr::allocator<int, Pool> Alloc;
  thrust::device_memory_resource upstream;
  Pool pool(&upstream);
  Alloc alloc(&pool);
  {
    thrust::device_vector<int, Alloc> v(alloc);
    v.resize(1000, 7);
    v.push_back(9);
    ASSERT_EQUAL(v.size(), (std::size_t)1001);
    ASSERT_EQUAL(thrust::reduce(v.begin(), v.end()), 7009);
    thrust::host_vector<int> h = v;
    ASSERT_EQUAL(h[1000], 9);
    thrust::device_vector<int, Alloc> w(5, 3, alloc);
    ASSERT_TRUE(v.get_allocator() == w.get_allocator());
    thrust::sort(v.begin(), v.end(), thrust::greater<int>());
    ASSERT_EQUAL((int)v[0], 9);
  }
  ASSERT_TRUE(pool.upstream_allocations() >= 1);
  Alloc::rebind<double>::other dalloc(alloc);
  auto p = dalloc.allocate(10);
  dalloc.deallocate(p, 10);
  thrust::device_allocator<float> a1, a2;
  ASSERT_TRUE(a1 == a2);
  thrust::device_vector<float> plain(10, 1.5f);  // the default allocator: the library's pool
  ASSERT_EQUAL(thrust::reduce(plain.begin(), plain.end()), 15.0f);
  ASSERT_TRUE(thrust::system::cdna4::pool_memory_resource::bytes_held() > 0);
}
DECLARE_UNITTEST(TestDeviceVectorWithPoolAllocator);

// examples/cuda/custom_temporary_allocation.cu:20-130: a caching allocator for temporaries
struct cached_allocator {
  typedef char value_type;
  std::multimap<std::ptrdiff_t, char*> free_blocks;
  std::map<char*, std::ptrdiff_t> allocated_blocks;
  int hits = 0, misses = 0;
  char* allocate(std::ptrdiff_t num_bytes) {
    char* result = nullptr;
    auto block = free_blocks.find(num_bytes);
    if (block != free_blocks.end()) {
      ++hits;
      result = block->second;
      free_blocks.erase(block);
    } else {
      ++misses;
      void* p = nullptr;
      if (thrust_cdna4_malloc_direct(&p, (std::size_t)num_bytes) != 0) throw std::bad_alloc();
      result = static_cast<char*>(p);
    }
    allocated_blocks.insert(std::make_pair(result, num_bytes));
    return result;
  }
  void deallocate(char* ptr, std::size_t) {
    auto it = allocated_blocks.find(ptr);
    const std::ptrdiff_t n = it->second;
    allocated_blocks.erase(it);
    free_blocks.insert(std::make_pair(n, ptr));
  }
  ~cached_allocator() {
    for (auto& b : free_blocks) thrust_cdna4_free_direct(b.second);
    for (auto& b : allocated_blocks) thrust_cdna4_free_direct(b.first);
  }
};
void TestTemporaryStorageFromUserAllocator() {
  const std::size_t n = 1 << 20;
  thrust::host_vector<int> h = unittest::random_integers<int>(n);
  cached_allocator alloc;
  for (int round = 0; round < 3; round++) {
    thrust::device_vector<int> d = h, out(n);
    thrust::sort(thrust::cdna4::par(alloc), d.begin(), d.end());
    thrust::inclusive_scan(thrust::cdna4::par(alloc), d.begin(), d.end(), out.begin());
    thrust::host_vector<int> sorted = h;
    std::sort(sorted.begin(), sorted.end());
    ASSERT_EQUAL(sorted, d);
    thrust::host_vector<int> scanned(n);
    thrust::inclusive_scan(sorted.begin(), sorted.end(), scanned.begin());
    ASSERT_EQUAL(scanned, out);
  }
  ASSERT_TRUE(alloc.misses >= 1 && alloc.misses <= 2);  // one block size per algorithm, allocated once
  ASSERT_TRUE(alloc.hits >= 4);                          // and reused in the later rounds
  ASSERT_TRUE(alloc.allocated_blocks.empty());
}
DECLARE_UNITTEST(TestTemporaryStorageFromUserAllocator);

// testing/mr_disjoint_pool.cu:120-260: the same caching behaviour with the pool's records in
// memory of a second resource, which the test sees being used
void TestDisjointPool() {
  thrust::mr::new_delete_resource heap;
  tracking_resource<thrust::mr::new_delete_resource> book(&heap);
  {
    thrust::device_memory_resource dev;
    tracking_resource<thrust::device_memory_resource> up(&dev);
    typedef thrust::mr::disjoint_unsynchronized_pool_resource<tracking_resource<thrust::device_memory_resource>,
                                                               tracking_resource<thrust::mr::new_delete_resource>> Pool;
    thrust::mr::pool_options opt = thrust::mr::unsynchronized_pool_resource<thrust::mr::new_delete_resource>::get_default_options();
    opt.smallest_block_size = 256;
    opt.largest_block_size = 1 << 16;
    Pool pool(&up, &book, opt);
    ASSERT_TRUE(book.allocations > 0);  // the size-class table lives in the bookkeeper's memory
    thrust::device_ptr<void> a = pool.allocate(1000, 256);
    const int chunk_allocations = up.allocations;
    ASSERT_EQUAL(chunk_allocations, 1);
    pool.deallocate(a, 1000, 256);
    thrust::device_ptr<void> b = pool.allocate(900, 256);  // the same class: served from the cache
    ASSERT_TRUE(a == b);
    ASSERT_EQUAL(up.allocations, chunk_allocations);
    pool.deallocate(b, 900, 256);
    thrust::device_ptr<void> big = pool.allocate(1 << 20, 256);  // oversized: straight from upstream, cached afterwards
    pool.deallocate(big, 1 << 20, 256);
    ASSERT_TRUE(pool.allocate(1 << 20, 256) == big);
    pool.deallocate(big, 1 << 20, 256);
    // a device_vector over the pool
    typedef thrust::mr::allocator<int, Pool> Alloc;
    thrust::device_vector<int, Alloc> v(1000, 2, Alloc(&pool));
    ASSERT_EQUAL(thrust::reduce(v.begin(), v.end()), 2000);
    pool.release();
    ASSERT_EQUAL(up.allocations, up.deallocations + 0);
  }
  ASSERT_EQUAL(book.allocations, book.deallocations);  // the records were returned too
  ASSERT_EQUAL(book.live_bytes, std::size_t(0));
}
DECLARE_UNITTEST(TestDisjointPool);

// testing/mr_pool.cu (synchronized), mr_disjoint_pool.cu (synchronized): several threads on one pool
template <class Pool>
void hammer(Pool& pool) {
  std::vector<std::thread> threads;
  std::vector<int> ok(8, 0);
  for (int t = 0; t < 8; t++)
    threads.emplace_back([&pool, &ok, t] {
      bool good = true;
      for (int i = 0; i < 200; i++) {
        const std::size_t bytes = 64 + 64 * ((i * 7 + t) % 50);
        void* p = pool.allocate(bytes, 64);
        good = good && p != nullptr;
        static_cast<char*>(p)[bytes - 1] = (char)t;
        void* q = pool.allocate(bytes, 64);
        good = good && q != p;
        pool.deallocate(p, bytes, 64);
        pool.deallocate(q, bytes, 64);
      }
      ok[t] = good;
    });
  for (auto& th : threads) th.join();
  for (int t = 0; t < 8; t++) ASSERT_TRUE(ok[t]);
}
void TestSynchronizedAndThreadLocalPools() {
  thrust::mr::new_delete_resource heap;
  thrust::mr::synchronized_pool_resource<thrust::mr::new_delete_resource> sync(&heap);
  hammer(sync);
  sync.release();
  thrust::mr::disjoint_synchronized_pool_resource<thrust::mr::new_delete_resource, thrust::mr::new_delete_resource> dsync(&heap, &heap);
  hammer(dsync);
  // one pool per thread: the same object within a thread, another one on another thread (a
  // thread's pool lives until the thread ends, so its upstream is the global resource object)
  thrust::mr::new_delete_resource* global = thrust::mr::get_global_resource<thrust::mr::new_delete_resource>();
  auto& mine = thrust::mr::tls_pool(global);
  ASSERT_TRUE(&mine == &thrust::mr::tls_pool<thrust::mr::new_delete_resource>());
  void* theirs = nullptr;
  std::thread([&] { theirs = &thrust::mr::tls_pool(global); }).join();
  ASSERT_TRUE(theirs != nullptr && theirs != (void*)&mine);
  void* p = mine.allocate(100, 64);
  mine.deallocate(p, 100, 64);
  ASSERT_TRUE(mine.allocate(100, 64) == p);
  mine.deallocate(p, 100, 64);
  auto& dmine = thrust::mr::disjoint_tls_pool(global, global);
  void* q = dmine.allocate(100, 64);
  dmine.deallocate(q, 100, 64);
}
DECLARE_UNITTEST(TestSynchronizedAndThreadLocalPools);

// examples/mr_basic.cu:38-60, testing/allocator.cu: one allocator type over resources chosen at run time
void TestPolymorphicAdaptorAndFancyPointerResource() {
  thrust::mr::new_delete_resource heap;
  tracking_resource<thrust::mr::new_delete_resource> tracked(&heap);
  thrust::mr::polymorphic_adaptor_resource<void*> adaptor(&tracked);
  typedef thrust::mr::polymorphic_allocator<int, void*> Alloc;
  Alloc alloc(&adaptor);
  {
    thrust::host_vector<int, Alloc> v(alloc);
    for (int i = 0; i < 100; i++) v.push_back(i);
    ASSERT_EQUAL(v.back(), 99);
    ASSERT_TRUE(tracked.allocations > 0);
  }
  ASSERT_EQUAL(tracked.allocations, tracked.deallocations);
  thrust::mr::polymorphic_adaptor_resource<void*> same(&tracked), other(&heap);
  ASSERT_TRUE(adaptor == same);
  ASSERT_TRUE(!(adaptor == other));
  // device memory through the adaptor
  thrust::device_memory_resource dev;
  thrust::mr::polymorphic_adaptor_resource<thrust::device_ptr<void>> dadaptor(&dev);
  typedef thrust::mr::polymorphic_allocator<int, thrust::device_ptr<void>> DAlloc;
  thrust::device_vector<int, DAlloc> d(100, 3, DAlloc(&dadaptor));
  ASSERT_EQUAL(thrust::reduce(d.begin(), d.end()), 300);
  // a host resource seen through device_ptr and back
  thrust::mr::fancy_pointer_resource<thrust::mr::new_delete_resource, thrust::device_ptr<void>> fancy(&heap);
  thrust::device_ptr<void> fp = fancy.allocate(64, 16);
  ASSERT_TRUE(fp.get() != nullptr);
  fancy.deallocate(fp, 64, 16);
  thrust::device_ptr_memory_resource<thrust::device_memory_resource> dpr;
  thrust::device_ptr<void> dp = dpr.allocate(256, 256);
  ASSERT_TRUE(dp.get() != nullptr);
  dpr.deallocate(dp, 256, 256);
  thrust::mr::validator<thrust::host_memory_resource> check1;
  thrust::mr::validator2<thrust::device_memory_resource, thrust::mr::new_delete_resource> check2;
  (void)check1; (void)check2;
}
DECLARE_UNITTEST(TestPolymorphicAdaptorAndFancyPointerResource);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }
