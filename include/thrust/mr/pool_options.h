// thrust::mr::pool_options (thrust/mr/pool_options.h).
#pragma once
#include <cstddef>

namespace thrust { namespace mr {
struct pool_options {
  std::size_t min_blocks_per_chunk = 16;          // blocks carved from one upstream allocation, at least
  std::size_t min_bytes_per_chunk = 1024;         // an upstream allocation is at least this large
  std::size_t max_blocks_per_chunk = std::size_t(1) << 20;
  std::size_t max_bytes_per_chunk = std::size_t(1) << 30;
  std::size_t smallest_block_size = alignof(std::max_align_t);  // a power of two
  std::size_t largest_block_size = std::size_t(1) << 20;        // a power of two; larger requests go upstream
  std::size_t alignment = 256;                    // of every block the pool hands out
  bool cache_oversized = true;                    // keep larger-than-largest blocks for reuse
  std::size_t cached_size_cutoff_factor = 16;     // a cached oversized block serves requests down to size / factor
  bool validate() const {
    const auto pow2 = [](std::size_t x) { return x && !(x & (x - 1)); };
    return pow2(smallest_block_size) && pow2(largest_block_size) && pow2(alignment) && smallest_block_size <= largest_block_size &&
           min_blocks_per_chunk <= max_blocks_per_chunk && min_bytes_per_chunk <= max_bytes_per_chunk && min_blocks_per_chunk > 0;
  }
};
}}  // namespace thrust::mr
