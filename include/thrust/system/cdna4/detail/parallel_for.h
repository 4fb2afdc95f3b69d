// Generic-functor building blocks of the cdna4 system: parallel_for and reduce as kernel
// templates (thrust/system/cuda/detail/parallel_for.h:70-174, reduce.h:152-669, :947-971).
// They carry user functors, so the translation unit that instantiates them is compiled by
// hipcc (--offload-arch=gfx950) and the functors' operator() must be __host__ __device__.
// for_each, transform, sequence, transform_reduce, reduce and count_if in the public headers are
// thin wrappers over these two; copy_if, remove_if and unique over the select engine below.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/cdna4/detail/parallel_for.h holds device kernel templates: compile with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdint>
#include <type_traits>
#include <thrust/system/cdna4/detail/core.h>

namespace thrust { namespace system { namespace cdna4 { namespace detail { namespace generic {

constexpr int kBlock = 256;
constexpr int kItems = 4;  // indices per thread, strided by the workgroup size: a wave touches contiguous elements

// f(i) for every i in [0, n)
template <class F>
__global__ __launch_bounds__(kBlock) void parallel_for_kernel(std::int64_t n, F f) {
  const std::int64_t base = (std::int64_t)blockIdx.x * (kBlock * kItems) + threadIdx.x;
#pragma unroll
  for (int k = 0; k < kItems; k++) {
    const std::int64_t i = base + (std::int64_t)k * kBlock;
    if (i < n) f(i);
  }
}

template <class F>
void parallel_for(void* stream, std::int64_t n, F f) {
  if (n <= 0) return;
  const std::int64_t blocks = (n + kBlock * kItems - 1) / (kBlock * kItems);
  hipLaunchKernelGGL((parallel_for_kernel<F>), dim3((unsigned)blocks), dim3(kBlock), 0, static_cast<hipStream_t>(stream), n, f);
  throw_on_error((int)hipGetLastError(), "parallel_for: launch");
}

// ---------------------------------------------------------------------------------------
// reduce: workgroup partials, then one workgroup over the partials.  `op` must be associative
// and commutative (the order of combination is unspecified, as in the reference); no identity
// is needed: threads without an element do not take part.
// ---------------------------------------------------------------------------------------
template <class T, class Op>
__device__ inline T block_reduce(T v, int valid_threads, Op op) {
  __shared__ typename std::aligned_storage<sizeof(T), alignof(T)>::type raw[kBlock];
  T* s = reinterpret_cast<T*>(raw);
  const int tid = threadIdx.x;
  s[tid] = v;
  __syncthreads();
#pragma unroll
  for (int stride = kBlock / 2; stride > 0; stride >>= 1) {
    if (tid < stride && tid + stride < valid_threads) {
      v = op(v, s[tid + stride]);
      s[tid] = v;
    }
    __syncthreads();
  }
  return v;  // the total, in thread 0
}

// partial[b] = op-reduction of unary(i) over the indices of workgroup b; every workgroup owns at
// least one index (the host sizes the grid so)
template <class T, class Unary, class Op>
__global__ __launch_bounds__(kBlock) void reduce_partials_kernel(std::int64_t n, Unary unary, Op op, T* partial) {
  const std::int64_t stride = (std::int64_t)gridDim.x * kBlock;
  std::int64_t i = (std::int64_t)blockIdx.x * kBlock + threadIdx.x;
  const std::int64_t first = (std::int64_t)blockIdx.x * kBlock;
  const int valid = (int)(n - first < kBlock ? n - first : kBlock);
  T acc{};
  if (i < n) {
    acc = unary(i);
    i += stride;
    for (; i + 3 * stride < n; i += 4 * stride) {  // four independent loads in flight
      const T a = unary(i), b = unary(i + stride), c = unary(i + 2 * stride), d = unary(i + 3 * stride);
      acc = op(op(acc, a), op(op(b, c), d));
    }
    for (; i < n; i += stride) acc = op(acc, unary(i));
  }
  acc = block_reduce(acc, valid, op);
  if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

// out[0] = op(init, partial[0] (+) ... (+) partial[count-1])
template <class T, class Op>
__global__ __launch_bounds__(kBlock) void reduce_final_kernel(const T* partial, int count, T init, Op op, T* out) {
  if (count <= 0) {  // an empty range reduces to init
    if (threadIdx.x == 0) out[0] = init;
    return;
  }
  T acc{};
  int i = threadIdx.x;
  if (i < count) {
    acc = partial[i];
    for (i += kBlock; i < count; i += kBlock) acc = op(acc, partial[i]);
  }
  acc = block_reduce(acc, count < kBlock ? count : kBlock, op);
  if (threadIdx.x == 0) out[0] = op(init, acc);
}

// Stores op(init, unary(0) (+) ... (+) unary(n-1)) at device address out, in stream order and
// without waiting (the asynchronous reductions; n == 0 stores init).
template <class T, class Unary, class Op>
void transform_reduce_into(void* stream_, std::int64_t n, Unary unary, T init, Op op, T* out) {
  static_assert(thrust::detail::is_bytewise_movable<T>::value, "cdna4 reduce: the result type must be movable as bytes");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  std::int64_t blocks = (n + kBlock - 1) / kBlock;
  const std::int64_t enough = 2048;
  if (blocks > enough) blocks = enough;
  temporary_storage tmp((std::size_t)(blocks > 0 ? blocks : 1) * sizeof(T), stream_);
  T* partial = static_cast<T*>(tmp.data());
  if (blocks > 0)
    hipLaunchKernelGGL((reduce_partials_kernel<T, Unary, Op>), dim3((unsigned)blocks), dim3(kBlock), 0, s, n, unary, op, partial);
  hipLaunchKernelGGL((reduce_final_kernel<T, Op>), dim3(1), dim3(kBlock), 0, s, partial, (int)blocks, init, op, out);
  throw_on_error((int)hipGetLastError(), "reduce: launch");
}

// Returns op(init, unary(0) (+) ... (+) unary(n-1)); blocks until the value is on the host
// (thrust/system/cuda/detail/reduce.h:947-971 does the same).
template <class T, class Unary, class Op>
T transform_reduce(void* stream_, std::int64_t n, Unary unary, T init, Op op) {
  static_assert(thrust::detail::is_bytewise_movable<T>::value, "cdna4 reduce: the result type must be movable as bytes");
  if (n <= 0) return init;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  std::int64_t blocks = (n + kBlock - 1) / kBlock;  // every workgroup gets at least one index
  const std::int64_t enough = 2048;                  // 8 workgroups per CU
  if (blocks > enough) blocks = enough;
  temporary_storage tmp((std::size_t)(blocks + 1) * sizeof(T), stream_);
  T* partial = static_cast<T*>(tmp.data());
  T* out = partial + blocks;
  hipLaunchKernelGGL((reduce_partials_kernel<T, Unary, Op>), dim3((unsigned)blocks), dim3(kBlock), 0, s, n, unary, op, partial);
  hipLaunchKernelGGL((reduce_final_kernel<T, Op>), dim3(1), dim3(kBlock), 0, s, partial, (int)blocks, init, op, out);
  throw_on_error((int)hipGetLastError(), "reduce: launch");
  T result;
  throw_on_error(thrust_cdna4_read_back(&result, out, sizeof(T), stream_), "reduce: read back");
  return result;
}

// ---------------------------------------------------------------------------------------
// select: stable compaction of the indices i in [0, n) that an operation keeps, in one pass
// (the shape of the reference's select engine, thrust/system/cuda/detail/copy_if.h:221-520, on
// 64-wide wavefronts).  The operation supplies
//     typedef ... item;                               what travels from the load to the store
//     item load(int64 i, bool& keep) const;           reads element i and decides
//     void store(const item&, int64 position) const;  writes a kept element
//     static const bool rejects;                      true: the others go to store_rejected(item,
//                                                     position among the rejected) — partition
// A tile loads its elements (all loads of a thread in flight together: load() must not branch on
// what it reads), ranks the kept ones inside the tile (wave ballots + a table of (row, wave)
// counts in LDS, scanned by wave 0), learns how many elements the tiles before it kept from a
// chain of tile descriptors (decoupled look-back, 64 descriptors per round, one per lane of
// wave 0) and stores from registers.  copy_if, remove_if, unique and unique_by_key are such
// operations.  Traffic: the inputs once, the kept outputs once.
//
// A descriptor is one 64-bit word, status in bits 63:62 (0 empty, 1 the tile's own count,
// 2 the count of all tiles up to and including it) and the count below, written and read with
// relaxed agent-scope atomics: the value travels inside the word, so no fence is needed.
// Tiles take their index from a ticket counter, so every tile a waiting tile looks back at has
// started already and the wait ends.  One same-address atomic costs about 12 ns of the whole
// device's time, which is why a tile is 128 KiB of items.  (A persistent variant that asks for its
// next ticket behind the loads of the current tile was measured 20 % slower: the ticket's latency
// is not what bounds the kernel — with nothing kept, hence no memory traffic at all, 8192 tiles
// still take 0.15 ms of ticket, barriers and look-back.)
// ---------------------------------------------------------------------------------------
#ifndef THRUST_CDNA4_SELECT_BLOCK
#define THRUST_CDNA4_SELECT_BLOCK 1024
#endif
constexpr int kSelBlock = THRUST_CDNA4_SELECT_BLOCK;
constexpr int kSelWaves = kSelBlock / 64;
constexpr unsigned long long kSelValueMask = (1ull << 62) - 1ull;
// rows of kSelBlock items per tile: 128 bytes of items per thread, 4 to 32 rows
constexpr int select_rows(std::size_t item_bytes) {
  return item_bytes <= 4 ? 32 : item_bytes <= 8 ? 16 : item_bytes <= 16 ? 8 : 4;
}
// An operation may ask for another number of rows with `static constexpr int rows` (at most 64:
// the kept rows of a thread are one 64-bit mask).  copy_if / remove_if on items of up to 4 bytes
// take 64: the tile's fixed costs (ticket, barriers, look-back) are paid half as often, 0.413 →
// 0.381 ms for 2^28 ints, and the kernel still fits its 128 registers (112); unique's operation
// does not (128 and spills: 3 % slower), so it stays at 32.  unique_by_key on 4-byte keys with
// 4-byte values (8-byte items) takes 32 rows instead of 16, on one workgroup per CU instead of two:
// 0.626 → 0.578 ms; copy_if on 8-byte items likewise.
template <class...> struct select_void { typedef void type; };
template <class Op, class = void>
struct select_rows_of { static constexpr int value = select_rows(sizeof(typename Op::item)); };
template <class Op>
struct select_rows_of<Op, typename select_void<decltype(Op::rows)>::type> { static constexpr int value = Op::rows; };
// Register budget: 32 rows of 4-byte items need about 72 registers (one workgroup per CU);
// 8- to 32-byte items fit 64 registers, and the second workgroup per CU is worth 12 %.
#ifndef THRUST_CDNA4_SELECT_WPE4
#define THRUST_CDNA4_SELECT_WPE4 4
#endif
constexpr int select_waves_per_simd(std::size_t item_bytes) { return item_bytes > 4 && item_bytes <= 32 ? 8 : THRUST_CDNA4_SELECT_WPE4; }

// more than 128 bytes of items per thread: one workgroup per CU on the full register budget
template <class Op>
struct select_waves_of {
  static constexpr int value = select_rows_of<Op>::value * sizeof(typename Op::item) > 128
                                   ? 4 : select_waves_per_simd(sizeof(typename Op::item));
};
// words[0, tiles) are the descriptors, words[tiles] the ticket counter, words[tiles + 1] the result
template <class Word>
__global__ __launch_bounds__(256) void select_init_kernel(Word* words, std::int64_t count) {
  const std::int64_t i = (std::int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < count) words[i] = Word(0);
}

template <bool REJECTS> struct select_rejected {
  template <class Op, class Item> __device__ static void store(const Op& op, const Item& x, std::int64_t pos) { op.store_rejected(x, pos); }
};
template <> struct select_rejected<false> {
  template <class Op, class Item> __device__ static void store(const Op&, const Item&, std::int64_t) {}
};

template <class Op>
__global__ __launch_bounds__(kSelBlock)
__attribute__((amdgpu_waves_per_eu(select_waves_of<Op>::value, select_waves_of<Op>::value)))
void select_kernel(std::int64_t n, Op op, unsigned long long* words, std::int64_t tiles) {
  typedef typename Op::item Item;
  constexpr int ROWS = select_rows_of<Op>::value;
  static_assert(ROWS <= 64 && (ROWS * kSelWaves) % 64 == 0, "one 64-bit mask of kept rows; whole lanes of (row, wave) cells");
  constexpr int TILE = kSelBlock * ROWS;
  constexpr int CELLS = ROWS * kSelWaves;  // (row, wave) counts
  constexpr int PER_LANE = CELLS / 64;     // cells each lane of wave 0 scans
  __shared__ unsigned s_cnt[CELLS];        // kept in (row, wave), then its exclusive prefix in the tile
  __shared__ unsigned long long s_tile, s_prefix;
  const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
  if (threadIdx.x == 0)
    s_tile = __hip_atomic_fetch_add(&words[tiles], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const std::int64_t tile = (std::int64_t)s_tile;
  const std::int64_t base = tile * TILE + threadIdx.x;
  Item items[ROWS];
  unsigned long long mine = 0;  // bit j: row j's element is kept
  if ((tile + 1) * TILE <= n) {
#pragma unroll
    for (int j = 0; j < ROWS; j++) {
      bool keep;
      items[j] = op.load(base + (std::int64_t)j * kSelBlock, keep);
      mine |= (unsigned long long)(keep ? 1u : 0u) << j;
    }
  } else {
#pragma unroll
    for (int j = 0; j < ROWS; j++) {
      // the last tile: every thread loads (the last element where it has none of its own), so
      // that the loads stay independent of each other; what it loaded there is never kept
      const std::int64_t i = base + (std::int64_t)j * kSelBlock;
      bool keep;
      items[j] = op.load(i < n ? i : n - 1, keep);
      mine |= (unsigned long long)(keep && i < n ? 1u : 0u) << j;
    }
  }
#pragma unroll
  for (int j = 0; j < ROWS; j++) {
    const unsigned long long m = __builtin_amdgcn_ballot_w64((mine >> j) & 1u);
    if (lane == 0) s_cnt[j * kSelWaves + wave] = (unsigned)__builtin_popcountll(m);
  }
  __syncthreads();
  if (wave == 0) {
    unsigned c[PER_LANE], sum = 0;
#pragma unroll
    for (int q = 0; q < PER_LANE; q++) {
      c[q] = s_cnt[lane * PER_LANE + q];
      sum += c[q];
    }
    unsigned inc = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const unsigned up = __shfl_up(inc, d, 64);
      if (lane >= d) inc += up;
    }
    unsigned run = inc - sum;
#pragma unroll
    for (int q = 0; q < PER_LANE; q++) {
      s_cnt[lane * PER_LANE + q] = run;
      run += c[q];
    }
    const unsigned long long total = (unsigned long long)__shfl(inc, 63, 64);
    unsigned long long prefix = 0;  // kept by all tiles before this one
    if (tile > 0) {
      if (lane == 0) __hip_atomic_store(&words[tile], (1ull << 62) | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      std::int64_t nearest = tile - 1;
      for (;;) {
        const std::int64_t t = nearest - lane;  // lane 0 looks at the nearest tile before this one
        const unsigned long long w =
            t >= 0 ? __hip_atomic_load(&words[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : (2ull << 62);
        const unsigned status = (unsigned)(w >> 62);
        const unsigned long long full = __builtin_amdgcn_ballot_w64(status == 2u);
        const unsigned long long empty = __builtin_amdgcn_ballot_w64(status == 0u);
        // lanes up to and including the nearest complete descriptor contribute
        const unsigned long long use = full ? ((full & (0ull - full)) << 1) - 1ull : ~0ull;
        if (empty & use) {
          __builtin_amdgcn_s_sleep(1);
          continue;
        }
        unsigned long long v = ((use >> lane) & 1ull) ? (w & kSelValueMask) : 0ull;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
        prefix += v;
        if (full) break;
        nearest -= 64;
      }
    }
    if (lane == 0) {
      __hip_atomic_store(&words[tile], (2ull << 62) | (prefix + total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_prefix = prefix;
      if (tile == tiles - 1) words[tiles + 1] = prefix + total;
    }
  }
  __syncthreads();
  const std::int64_t tile_off = (std::int64_t)s_prefix;
#pragma unroll
  for (int j = 0; j < ROWS; j++) {
    // kept elements before this one in the whole input; the rank inside the row's wavefront is
    // balloted again rather than kept in registers across the look-back
    const unsigned long long m = __builtin_amdgcn_ballot_w64((mine >> j) & 1u);
    const unsigned below = __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
    const std::int64_t before = tile_off + s_cnt[j * kSelWaves + wave] + below;
    const std::int64_t i = base + (std::int64_t)j * kSelBlock;
    if ((mine >> j) & 1u)
      op.store(items[j], before);
    else if (Op::rejects && i < n)
      select_rejected<Op::rejects>::store(op, items[j], i - before);  // rejected elements before this one
  }
}

// Returns the number of kept elements; blocks until it is known (the callers return an end
// iterator that depends on it, as the reference's do).
template <class Op>
std::int64_t select(void* stream_, std::int64_t n, Op op) {
  if (n <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  constexpr std::int64_t kTile = (std::int64_t)kSelBlock * select_rows_of<Op>::value;
  const std::int64_t tiles = (n + kTile - 1) / kTile;
  temporary_storage tmp((std::size_t)(tiles + 2) * sizeof(unsigned long long), stream_);
  unsigned long long* words = static_cast<unsigned long long*>(tmp.data());
  hipLaunchKernelGGL((select_init_kernel<unsigned long long>), dim3((unsigned)((tiles + 2 + 255) / 256)), dim3(256), 0, s, words, tiles + 2);
  hipLaunchKernelGGL((select_kernel<Op>), dim3((unsigned)tiles), dim3(kSelBlock), 0, s, n, op, words, tiles);
  throw_on_error((int)hipGetLastError(), "select: launch");
  unsigned long long kept = 0;
  throw_on_error(thrust_cdna4_read_back(&kept, words + tiles + 1, sizeof(kept), stream_), "select: read back");
  return (std::int64_t)kept;
}

}}}}}  // namespace thrust::system::cdna4::detail::generic
