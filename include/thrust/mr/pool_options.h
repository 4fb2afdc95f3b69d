// thrust::mr::pool_options (thrust/mr/pool_options.h).
#pragma once
#include <cstddef>

namespace thrust { namespace mr {
// All sizes start at zero, as in the reference: a default-constructed object is not valid; the
// pools' get_default_options() return the working defaults (default_pool_options below).
struct pool_options {
  std::size_t min_blocks_per_chunk = 0;           // blocks carved from one upstream allocation, at least
  std::size_t min_bytes_per_chunk = 0;            // an upstream allocation is at least this large
  std::size_t max_blocks_per_chunk = 0;
  std::size_t max_bytes_per_chunk = 0;
  std::size_t smallest_block_size = 0;            // a power of two
  std::size_t largest_block_size = 0;             // a power of two; larger requests go upstream
  std::size_t alignment = 0;                      // of every block the pool hands out; a power of two
  bool cache_oversized = false;                   // keep larger-than-largest blocks for reuse
  std::size_t cached_size_cutoff_factor = 0;      // a cached oversized block serves requests down to size / factor
  std::size_t cached_alignment_cutoff_factor = 0;
  // the consistency rules of thrust/mr/pool_options.h:97-120
  bool validate() const {
    const auto pow2 = [](std::size_t x) { return (x & (x - 1)) == 0; };  // zero passes, as in the reference
    if (!pow2(smallest_block_size) || !pow2(largest_block_size) || !pow2(alignment)) return false;
    if (max_bytes_per_chunk == 0 || max_blocks_per_chunk == 0) return false;
    if (smallest_block_size == 0 || largest_block_size == 0) return false;
    if (min_blocks_per_chunk > max_blocks_per_chunk || min_bytes_per_chunk > max_bytes_per_chunk) return false;
    if (smallest_block_size > largest_block_size) return false;
    // the chunk sizes the block counts allow must meet the ones given in bytes
    if (min_blocks_per_chunk * smallest_block_size > max_bytes_per_chunk) return false;
    if (min_blocks_per_chunk * largest_block_size > max_bytes_per_chunk) return false;
    if (max_blocks_per_chunk * largest_block_size < min_bytes_per_chunk) return false;
    if (max_blocks_per_chunk * smallest_block_size < min_bytes_per_chunk) return false;
    if (alignment > smallest_block_size) return false;
    return true;
  }
};
namespace detail {
// Blocks of 256 bytes and up, 256-byte aligned (what device code coalesces on); chunk sizes as in
// the reference's defaults (thrust/mr/pool.h:77-97).
inline pool_options default_pool_options() {
  pool_options o;
  o.min_blocks_per_chunk = 16;
  o.min_bytes_per_chunk = 1024;
  o.max_blocks_per_chunk = std::size_t(1) << 20;
  o.max_bytes_per_chunk = std::size_t(1) << 30;
  o.smallest_block_size = 256;
  o.largest_block_size = std::size_t(1) << 20;
  o.alignment = 256;
  o.cache_oversized = true;
  o.cached_size_cutoff_factor = 16;
  o.cached_alignment_cutoff_factor = 16;
  return o;
}
}  // namespace detail
}}  // namespace thrust::mr
