// thrust::mr::unsynchronized_pool_resource (thrust/mr/pool.h:68-): a caching pool over any
// upstream resource.  Requests up to largest_block_size are rounded up to a power of two and
// served from per-size free lists that are refilled by carving one upstream chunk into blocks;
// larger requests go upstream one by one and, with cache_oversized, come back from a cache.
// Nothing returns to the upstream before release() or destruction.  Not thread safe, and not
// stream ordered: a block may be handed out again as soon as it is deallocated, so deallocate
// only after the work that uses the block has completed.
#pragma once
#include <algorithm>
#include <memory>
#include <cstddef>
#include <stdexcept>
#include <vector>
#include <thrust/mr/memory_resource.h>
#include <thrust/mr/pool_options.h>

namespace thrust { namespace mr {
namespace detail {
// byte arithmetic on the resource's pointer type
template <class Pointer> struct byte_pointer {
  static Pointer advance(Pointer p, std::size_t bytes) { return Pointer(static_cast<char*>(static_cast<void*>(p.get())) + bytes); }
};
template <> struct byte_pointer<void*> {
  static void* advance(void* p, std::size_t bytes) { return static_cast<char*>(p) + bytes; }
};
}  // namespace detail

namespace detail {
// Where a pool keeps its own records (free lists, chunk table): ordinary host memory ...
struct heap_bookkeeping {
  template <class T> struct alloc { typedef std::allocator<T> type; };
  template <class T> std::allocator<T> get() const { return std::allocator<T>(); }
};
// ... or memory of a resource the user names (the "disjoint" pools: the pooled memory itself is
// never touched, so it may be memory the host cannot address).  Defined in <thrust/mr/disjoint_pool.h>.
template <class Bookkeeper> struct resource_bookkeeping;

template <class Upstream, class Book>
class pool_core : public memory_resource<typename Upstream::pointer> {
 public:
  typedef typename Upstream::pointer pointer;
  static pool_options get_default_options() { return detail::default_pool_options(); }

  pool_core(Upstream* upstream, Book book, pool_options options)
      : upstream_(upstream), opt_(options), book_(book), free_(book.template get<free_list>()), chunks_(book.template get<chunk>()),
        oversized_(book.template get<big>()) {
    if (!opt_.validate()) throw std::invalid_argument("thrust::mr::pool_options: inconsistent");
    if (opt_.alignment == 0) opt_.alignment = alignof(std::max_align_t);  // left unset by the caller
    std::size_t classes = 1;
    for (std::size_t s = opt_.smallest_block_size; s < opt_.largest_block_size; s <<= 1) ++classes;
    free_.assign(classes, free_list(book.template get<pointer>()));
  }
  ~pool_core() override { release(); }
  pool_core(const pool_core&) = delete;
  pool_core& operator=(const pool_core&) = delete;

  // everything goes back to the upstream; blocks still handed out become invalid
  void release() {
    for (auto& c : chunks_) upstream_->deallocate(c.p, c.bytes, opt_.alignment);
    chunks_.clear();
    for (auto& f : free_) f.clear();
    for (auto& o : oversized_) upstream_->deallocate(o.p, o.bytes, opt_.alignment);
    oversized_.clear();
  }
  Upstream* upstream_resource() const { return upstream_; }
  std::size_t upstream_allocations() const { return upstream_calls_; }  // chunks + oversized blocks requested so far

  pointer do_allocate(std::size_t bytes, std::size_t alignment) override {
    if (alignment > opt_.alignment) throw std::bad_alloc();  // blocks are opt_.alignment-aligned
    if (bytes == 0) bytes = 1;
    if (bytes > opt_.largest_block_size) return allocate_oversized(bytes);
    std::size_t size = opt_.smallest_block_size, cls = 0;
    while (size < bytes) { size <<= 1; ++cls; }
    free_list& list = free_[cls];
    if (list.empty()) refill(list, size);
    pointer p = list.back();
    list.pop_back();
    return p;
  }
  void do_deallocate(pointer p, std::size_t bytes, std::size_t) override {
    if (bytes == 0) bytes = 1;
    if (bytes > opt_.largest_block_size) {
      for (auto& o : oversized_)
        if (o.p == p) {
          if (opt_.cache_oversized) { o.in_use = false; return; }
          upstream_->deallocate(o.p, o.bytes, opt_.alignment);
          o = oversized_.back();
          oversized_.pop_back();
          return;
        }
      throw std::invalid_argument("thrust::mr::pool: deallocate of a block this pool did not allocate");
    }
    std::size_t size = opt_.smallest_block_size, cls = 0;
    while (size < bytes) { size <<= 1; ++cls; }
    free_[cls].push_back(p);
  }

 private:
  struct chunk { pointer p; std::size_t bytes; };
  struct big { pointer p; std::size_t bytes; bool in_use; };
  typedef std::vector<pointer, typename Book::template alloc<pointer>::type> free_list;

  void refill(free_list& list, std::size_t size) {
    const std::size_t stride = std::max(size, opt_.alignment);  // keeps every block aligned
    std::size_t blocks = std::max(opt_.min_blocks_per_chunk, (opt_.min_bytes_per_chunk + stride - 1) / stride);
    blocks = std::min(blocks, opt_.max_blocks_per_chunk);
    blocks = std::max<std::size_t>(1, std::min(blocks, opt_.max_bytes_per_chunk / stride));
    const std::size_t bytes = blocks * stride;
    pointer base = upstream_->allocate(bytes, opt_.alignment);
    ++upstream_calls_;
    chunks_.push_back(chunk{base, bytes});
    for (std::size_t b = blocks; b-- > 0;) list.push_back(detail::byte_pointer<pointer>::advance(base, b * stride));
  }
  pointer allocate_oversized(std::size_t bytes) {
    if (opt_.cache_oversized) {
      big* best = nullptr;
      for (auto& o : oversized_)
        if (!o.in_use && o.bytes >= bytes && (opt_.cached_size_cutoff_factor == 0 || o.bytes / opt_.cached_size_cutoff_factor <= bytes) && (!best || o.bytes < best->bytes)) best = &o;
      if (best) { best->in_use = true; return best->p; }
    }
    pointer p = upstream_->allocate(bytes, opt_.alignment);
    ++upstream_calls_;
    oversized_.push_back(big{p, bytes, true});
    return p;
  }

  Upstream* upstream_;
  pool_options opt_;
  Book book_;
  std::vector<free_list, typename Book::template alloc<free_list>::type> free_;
  std::vector<chunk, typename Book::template alloc<chunk>::type> chunks_;
  std::vector<big, typename Book::template alloc<big>::type> oversized_;
  std::size_t upstream_calls_ = 0;
};
}  // namespace detail

template <class Upstream>
class unsynchronized_pool_resource final : public detail::pool_core<Upstream, detail::heap_bookkeeping> {
  typedef detail::pool_core<Upstream, detail::heap_bookkeeping> core;
 public:
  static pool_options get_default_options() { return detail::default_pool_options(); }
  explicit unsynchronized_pool_resource(Upstream* upstream, pool_options options = get_default_options())
      : core(upstream, detail::heap_bookkeeping(), options) {}
  explicit unsynchronized_pool_resource(pool_options options = get_default_options())
      : core(get_global_resource<Upstream>(), detail::heap_bookkeeping(), options) {}
};
}}  // namespace thrust::mr
