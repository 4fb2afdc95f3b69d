// Stable comparison (merge) sort for gfx950, for keys or comparators the radix kernels cannot
// take: user-defined comparison functors, non-arithmetic trivially copyable keys.  This is
// the second branch of the reference's sort dispatch (thrust/system/cuda/detail/sort.h:59-205,
// :410-429, cub::DispatchMergeSort); semantics: thrust/system/detail/sequential/
// stable_merge_sort.inl (a stable sort: equal keys keep their input order).
//
// Unlike the radix path, the comparator is user code, so these are kernel TEMPLATES: the
// translation unit that instantiates them must be compiled by hipcc (--offload-arch=gfx950)
// and the comparator's operator() must be __host__ __device__.  Temporary storage comes from
// the library's stream-ordered pool.
//
//   1. block_sort_kernel   a workgroup of kBlock threads sorts a tile of kBlock*kIpt items (512
//                          threads; 8 items per thread for narrow keys alone, else 4: the
//                          per-thread search and serial merge are the critical path): every thread
//                          sorts its kIpt consecutive items in registers (odd-even transposition,
//                          stable), then log2(kBlock) rounds of merge-path merging through LDS.
//   2. merge_partition_kernel + merge_kernel, once per doubling of the run width: one thread
//                          per output tile finds where the tile starts in the two runs it
//                          merges (binary search on the merge path, ties to the left run);
//                          a workgroup then loads the two pieces into LDS, every thread merges
//                          its kIpt outputs, and the tile is written back with contiguous stores.
//      Values follow their keys through LDS by source index.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/cdna4/detail/merge_sort.h holds device kernel templates: compile with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <cstdint>
#include <type_traits>
#include <thrust/system/cdna4/detail/core.h>
#include <thrust/system/cdna4/detail/parallel_for.h>

namespace thrust { namespace system { namespace cdna4 { namespace detail { namespace merge {

#ifndef THRUST_CDNA4_MERGE_BLOCK
#define THRUST_CDNA4_MERGE_BLOCK 512
#endif
constexpr int kBlock = THRUST_CDNA4_MERGE_BLOCK;  // threads per workgroup
// Items per thread: a template parameter of the kernels, chosen by the host from the item size.
// Eight while key and value together take up to 8 bytes (the merge-path search is paid once per
// thread, so more items amortise it, and there is one pass fewer: 2^26 uint32 keys 3.4 ms against
// 4.0 ms, with uint32 values 3.8 against 4.2), four for wider items, whose tiles would crowd LDS.
#ifndef THRUST_CDNA4_MERGE_IPT_NARROW
#define THRUST_CDNA4_MERGE_IPT_NARROW 8
#endif
#ifndef THRUST_CDNA4_MERGE_IPT
#define THRUST_CDNA4_MERGE_IPT 4
#endif
template <class K, class V>
constexpr int items_per_thread() {
  return sizeof(K) + (std::is_empty<V>::value ? 0 : sizeof(V)) <= 8 ? THRUST_CDNA4_MERGE_IPT_NARROW : THRUST_CDNA4_MERGE_IPT;
}

struct no_value {};

// Items per thread of the tile sort: IPT, or IPT / 2 when two copies of keys and 16-bit positions
// and one of the values do not fit the 64 KiB of static LDS at IPT.  (Half a merge tile is the
// least the merge passes can start from: an output tile must lie within one pair of runs.)
template <class K, class V, int IPT>
constexpr int tile_sort_items() {
  constexpr std::size_t per_item = 2 * sizeof(K) + 4 + (std::is_same<V, no_value>::value ? 0 : sizeof(V));
  static_assert(per_item * kBlock * (IPT / 2) <= 65536, "cdna4 merge sort: half a tile does not fit LDS twice");
  return per_item * kBlock * IPT <= 65536 ? IPT : IPT / 2;
}

// A thread's kIpt consecutive items as one block: when the block is a whole number of 16-byte
// words it moves with 128-bit accesses (a wavefront then touches every byte of the lines it
// writes with one instruction instead of a quarter of them with each of four).  The copies are
// memcpys at the items' own alignment, for which the compiler emits those accesses on gfx950.
template <class T, int IPT>
struct alignas(16) item_block { T v[IPT]; };
template <class T, int IPT>
constexpr bool blockable() { return sizeof(item_block<T, IPT>) == sizeof(T) * IPT; }

// Number of items the first `diag` outputs of merge(a[0,na), b[0,nb)) take from a, with ties
// going to a (stability: a is the earlier run).
template <class K, class Compare>
__device__ inline int merge_path(const K* a, int na, const K* b, int nb, int diag, Compare comp) {
  int lo = diag > nb ? diag - nb : 0;
  int hi = diag < na ? diag : na;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (!comp(b[diag - 1 - mid], a[mid])) lo = mid + 1;  // a[mid] <= b[...]: a[mid] is among the first diag
    else hi = mid;
  }
  return lo;
}

// ---------------------------------------------------------------------------------------
// 1. Tile sort
// ---------------------------------------------------------------------------------------
// The rounds of the in-tile merge alternate between two LDS buffers: round r writes buffer r & 1
// and reads only that buffer, so a round never overwrites what the round before it may still be
// reading, and one workgroup barrier per round (between the writes and the reads) is enough.
template <int IPT, class K, class V, class Compare>
__global__ __launch_bounds__(kBlock) void block_sort_kernel(K* keys, V* values, std::int64_t n, Compare comp) {
  constexpr int kIpt = IPT, kTile = kBlock * IPT;
  static_assert((kIpt & (kIpt - 1)) == 0 && kTile <= 65536, "run widths double from kIpt; 16-bit positions in a tile");
  constexpr bool kHasValues = !std::is_same<V, no_value>::value;
  __shared__ K s_keys2[2][kTile];
  __shared__ std::uint16_t s_idx2[2][kTile];
  __shared__ typename std::conditional<kHasValues, V, char>::type s_vals[kHasValues ? kTile : 1];

  const int tid = threadIdx.x;
  const std::int64_t base = (std::int64_t)blockIdx.x * kTile;
  const int valid = (int)((n - base) < (std::int64_t)kTile ? (n - base) : (std::int64_t)kTile);

  // Items past the end of the input (last tile only) order after every real item; they are
  // recognised by their original position, which every item carries along.
  auto before = [&](const K& a, int ia, const K& b, int ib) -> bool {
    if (ib >= valid) return ia < valid;
    if (ia >= valid) return false;
    return comp(a, b);
  };

  K k[kIpt];
  int idx[kIpt];
  const bool whole = valid == kTile;
  if (whole && blockable<K, IPT>()) {
    item_block<K, IPT> blk;
    __builtin_memcpy(&blk, keys + base + tid * kIpt, sizeof(blk));
#pragma unroll
    for (int j = 0; j < kIpt; j++) {
      idx[j] = tid * kIpt + j;
      k[j] = blk.v[j];
    }
    if constexpr (kHasValues) {
#pragma unroll
      for (int j = 0; j < kIpt; j++) s_vals[idx[j]] = values[base + idx[j]];
    }
  } else
#pragma unroll
  for (int j = 0; j < kIpt; j++) {
    idx[j] = tid * kIpt + j;
    if (idx[j] < valid) {
      k[j] = keys[base + idx[j]];
      if constexpr (kHasValues) s_vals[idx[j]] = values[base + idx[j]];
    } else {
      k[j] = keys[base];  // any initialised value: never compared as a key
    }
  }

  // thread-local stable sort: odd-even transposition, swapping only strictly out-of-order pairs
#pragma unroll
  for (int round = 0; round < kIpt; round++) {
#pragma unroll
    for (int j = round & 1; j + 1 < kIpt; j += 2) {
      if (before(k[j + 1], idx[j + 1], k[j], idx[j])) {
        const K tk = k[j]; k[j] = k[j + 1]; k[j + 1] = tk;
        const int ti = idx[j]; idx[j] = idx[j + 1]; idx[j + 1] = ti;
      }
    }
  }

  // Merge runs of `width` items pairwise, doubling the width.  In a whole tile the comparator
  // alone orders the items (no padding to recognise), and the positions travel only when there
  // are values to fetch by them.  The serial merge is branch-free: one LDS read per output, of the
  // next item of whichever run the output came from, at a clamped index.
  auto rounds = [&](auto whole_tag) {
    constexpr bool kWhole = decltype(whole_tag)::value;
    constexpr bool kIdx = kHasValues || !kWhole;
    int round = 0;
    for (int width = kIpt; width < kTile; width *= 2, round ^= 1) {
      K* const s_keys = s_keys2[round];
      std::uint16_t* const s_idx = s_idx2[round];
#pragma unroll
      for (int j = 0; j < kIpt; j++) {
        s_keys[tid * kIpt + j] = k[j];
        if constexpr (kIdx) s_idx[tid * kIpt + j] = (std::uint16_t)idx[j];
      }
      __syncthreads();
      const int start = (tid * kIpt) & ~(2 * width - 1);
      const int diag = tid * kIpt - start;
      const K* a = s_keys + start;  // the right run follows the left one: b[i] == a[width + i]
      const std::uint16_t* ia = s_idx + start;
      int lo = diag > width ? diag - width : 0;
      int hi = diag < width ? diag : width;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        const int m = width + diag - 1 - mid;
        bool right_first;
        if constexpr (kWhole) right_first = comp(a[m], a[mid]);
        else right_first = before(a[m], ia[m], a[mid], ia[mid]);
        if (!right_first) lo = mid + 1;
        else hi = mid;
      }
      int pa = lo, pb = diag - lo;
      const int fa = pa < width ? pa : width - 1, fb = width + (pb < width ? pb : width - 1);
      K ka = a[fa], kb = a[fb];
      int xa = 0, xb = 0;
      if constexpr (kIdx) { xa = ia[fa]; xb = ia[fb]; }
#pragma unroll
      for (int j = 0; j < kIpt; j++) {
        bool right_first;
        if constexpr (kWhole) right_first = comp(kb, ka);
        else right_first = before(kb, xb, ka, xa);
        const bool take_a = pb >= width || (pa < width && !right_first);
        k[j] = take_a ? ka : kb;
        if constexpr (kIdx) idx[j] = take_a ? xa : xb;
        pa += take_a ? 1 : 0;
        pb += take_a ? 0 : 1;
        const int next = take_a ? (pa < width ? pa : width - 1) : width + (pb < width ? pb : width - 1);
        const K kn = a[next];
        ka = take_a ? kn : ka;
        kb = take_a ? kb : kn;
        if constexpr (kIdx) {
          const int xn = ia[next];
          xa = take_a ? xn : xa;
          xb = take_a ? xb : xn;
        }
      }
    }
  };
  if (whole) rounds(std::true_type{});
  else rounds(std::false_type{});

  // the first `valid` outputs are the real items, in order
  __syncthreads();
  if (whole && blockable<K, IPT>()) {
    item_block<K, IPT> blk;
#pragma unroll
    for (int j = 0; j < kIpt; j++) blk.v[j] = k[j];
    __builtin_memcpy(keys + base + tid * kIpt, &blk, sizeof(blk));
    if constexpr (kHasValues) {
      if (blockable<V, IPT>()) {
        item_block<V, IPT> vb;
#pragma unroll
        for (int j = 0; j < kIpt; j++) vb.v[j] = s_vals[idx[j]];
        __builtin_memcpy(values + base + tid * kIpt, &vb, sizeof(vb));
      } else {
#pragma unroll
        for (int j = 0; j < kIpt; j++) values[base + tid * kIpt + j] = s_vals[idx[j]];
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < kIpt; j++) {
    const int o = tid * kIpt + j;
    if (o < valid) {
      keys[base + o] = k[j];
      if constexpr (kHasValues) values[base + o] = s_vals[idx[j]];
    }
  }
}

// ---------------------------------------------------------------------------------------
// 2. One merge pass: runs of `width` items -> runs of 2*width
// ---------------------------------------------------------------------------------------
struct pair_geometry {
  std::int64_t a0, na, b0, nb, diag;
};
__device__ inline pair_geometry geometry_of(std::int64_t tile, std::int64_t width, std::int64_t n, int kTile) {
  pair_geometry g;
  const std::int64_t out0 = tile * kTile;
  const std::int64_t pstart = out0 / (2 * width) * (2 * width);
  g.a0 = pstart;
  const std::int64_t a1 = pstart + width < n ? pstart + width : n;
  const std::int64_t b1 = pstart + 2 * width < n ? pstart + 2 * width : n;
  g.na = a1 - g.a0;
  g.b0 = a1;
  g.nb = b1 - a1;
  g.diag = out0 - pstart;
  return g;
}

// splits[t] = how many items of the left run precede output tile t (binary search in global memory)
template <int IPT, class K, class Compare>
__global__ __launch_bounds__(256) void merge_partition_kernel(const K* keys, std::int64_t n, std::int64_t width,
                                                              std::int64_t ntiles, std::int64_t* splits,
                                                              Compare comp) {
  constexpr int kTile = kBlock * IPT;
  const std::int64_t t = (std::int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= ntiles) return;
  const pair_geometry g = geometry_of(t, width, n, kTile);
  const K* a = keys + g.a0;
  const K* b = keys + g.b0;
  std::int64_t lo = g.diag > g.nb ? g.diag - g.nb : 0;
  std::int64_t hi = g.diag < g.na ? g.diag : g.na;
  while (lo < hi) {
    const std::int64_t mid = (lo + hi) >> 1;
    if (!comp(b[g.diag - 1 - mid], a[mid])) lo = mid + 1;
    else hi = mid;
  }
  splits[t] = lo;
}

template <int IPT, class K, class V, class Compare>
__global__ __launch_bounds__(kBlock) void merge_kernel(const K* kin, const V* vin, K* kout, V* vout, std::int64_t n,
                                                       std::int64_t width, std::int64_t ntiles,
                                                       const std::int64_t* splits, Compare comp) {
  constexpr int kIpt = IPT, kTile = kBlock * IPT;
  constexpr bool kHasValues = !std::is_same<V, no_value>::value;
  __shared__ K s_keys[kTile];
  __shared__ typename std::conditional<kHasValues, V, char>::type s_vals[kHasValues ? kTile : 1];

  const int tid = threadIdx.x;
  const std::int64_t tile = blockIdx.x;
  const pair_geometry g = geometry_of(tile, width, n, kTile);
  const std::int64_t total = g.na + g.nb;                                 // outputs of the pair
  const int count = (int)(total - g.diag < kTile ? total - g.diag : kTile);  // outputs of this tile
  // left-run items before this tile and before the next one (the pair's last tile takes the rest)
  const std::int64_t sa0 = splits[tile];
  const bool last_of_pair = g.diag + kTile >= total;
  const std::int64_t sa1 = last_of_pair ? g.na : splits[tile + 1];
  const int na = (int)(sa1 - sa0);
  const int nb = count - na;

  // kIpt independent loads per thread, all in flight together: the index is clamped rather than
  // tested, because a load under a branch (or in a loop of unknown length) waits for the one
  // before it
  {
    K lk[kIpt];
    typename std::conditional<kHasValues, V, char>::type lv[kIpt];
#pragma unroll
    for (int u = 0; u < kIpt; u++) {
      const int i = tid + u * kBlock;
      const int ic = i < count ? i : count - 1;  // count >= 1: a tile is never empty
      const std::int64_t src = ic < na ? (g.a0 + sa0 + ic) : (g.b0 + (g.diag - sa0) + (ic - na));
      lk[u] = kin[src];
      if constexpr (kHasValues) lv[u] = vin[src];
    }
#pragma unroll
    for (int u = 0; u < kIpt; u++) {
      const int i = tid + u * kBlock;
      if (i < count) {
        s_keys[i] = lk[u];
        if constexpr (kHasValues) s_vals[i] = lv[u];
      }
    }
  }
  __syncthreads();

  const K* a = s_keys;
  const K* b = s_keys + na;
  int d = tid * kIpt;
  if (d > count) d = count;
  int pa = merge_path(a, na, b, nb, d, comp);
  int pb = d - pa;
  K k[kIpt];
  std::uint16_t src[kIpt];
  // serial merge with the two candidate keys held in registers: one LDS read per output
  // (the tile is never empty, so index 0 is always readable)
  K ka = a[pa < na ? pa : 0], kb = s_keys[pb < nb ? na + pb : 0];
#pragma unroll
  for (int j = 0; j < kIpt; j++) {  // branch-free; outputs past `count` are computed and not stored
    const bool take_a = pb >= nb || (pa < na && !comp(kb, ka));
    k[j] = take_a ? ka : kb;
    src[j] = (std::uint16_t)(take_a ? pa : na + pb);
    pa += take_a ? 1 : 0;
    pb += take_a ? 0 : 1;
    const int next = take_a ? (pa < na ? pa : 0) : (pb < nb ? na + pb : 0);
    const K kn = s_keys[next];
    ka = take_a ? kn : ka;
    kb = take_a ? kb : kn;
  }
  const std::int64_t out0 = tile * kTile;
  if (count == kTile) {  // a whole tile: every thread has kIpt outputs
    if (blockable<K, IPT>()) {
      item_block<K, IPT> blk;
#pragma unroll
      for (int j = 0; j < kIpt; j++) blk.v[j] = k[j];
      __builtin_memcpy(kout + out0 + d, &blk, sizeof(blk));
    } else {
#pragma unroll
      for (int j = 0; j < kIpt; j++) kout[out0 + d + j] = k[j];
    }
    if constexpr (kHasValues) {
      if (blockable<V, IPT>()) {
        item_block<V, IPT> blk;
#pragma unroll
        for (int j = 0; j < kIpt; j++) blk.v[j] = s_vals[src[j]];
        __builtin_memcpy(vout + out0 + d, &blk, sizeof(blk));
      } else {
#pragma unroll
        for (int j = 0; j < kIpt; j++) vout[out0 + d + j] = s_vals[src[j]];
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < kIpt; j++) {
    if (d + j < count) {
      kout[out0 + d + j] = k[j];
      if constexpr (kHasValues) vout[out0 + d + j] = s_vals[src[j]];
    }
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
inline std::size_t align256(std::size_t x) { return (x + 255) & ~std::size_t(255); }

// Whether tiles of K (and V) can live in the static LDS arrays of the kernels above: half a sort
// tile and a whole merge tile must fit 64 KiB, and LDS arrays cannot hold a type whose default
// constructor or destructor does anything.
template <class K, class V>
constexpr bool tiles_fit_lds() {
  constexpr bool has_values = !std::is_same<V, no_value>::value;
  constexpr std::size_t vsize = has_values ? sizeof(V) : 0;
  constexpr int IPT = items_per_thread<K, V>();
  return std::is_trivially_default_constructible<K>::value && std::is_trivially_destructible<K>::value &&
         std::is_trivially_default_constructible<V>::value && std::is_trivially_destructible<V>::value &&
         (sizeof(K) + vsize + 2) * kBlock * IPT <= 65536 && (2 * sizeof(K) + 4 + vsize) * kBlock * (IPT / 2) <= 65536;
}

template <class K, class V, class Compare>
void stable_sort_tiles(void* stream_, K* keys, V* values, std::int64_t n, Compare comp);

// Wide or non-trivial elements (the reference sorts keys and values of 8 KiB each,
// testing/stable_sort_by_key_large_keys_and_values.cu): their positions are sorted instead, under
// a comparison that reads the keys where they lie, and keys and values are then gathered once.
// Positions of equivalent keys stay in their order, so the sort is stable.
template <class I, class K, class Compare> struct compare_at {
  const K* keys; mutable Compare comp;
  __device__ bool operator()(I a, I b) const { return comp(keys[a], keys[b]); }
};
template <class I> struct iota_body {
  I* out;
  __device__ void operator()(std::int64_t i) const { out[i] = (I)i; }
};
template <class I, class T> struct gather_body {
  const T* in; const I* at; T* out;
  __device__ void operator()(std::int64_t i) const { out[i] = in[at[i]]; }
};
template <class I, class K, class V, class Compare>
void stable_sort_positions(void* stream_, K* keys, V* values, std::int64_t n, Compare comp) {
  constexpr bool kHasValues = !std::is_same<V, no_value>::value;
  const std::size_t ibytes = align256((std::size_t)n * sizeof(I));
  const std::size_t kbytes = align256((std::size_t)n * sizeof(K));
  const std::size_t vbytes = kHasValues ? align256((std::size_t)n * sizeof(V)) : 0;
  temporary_storage tmp(ibytes + kbytes + vbytes, stream_);
  char* t = static_cast<char*>(tmp.data());
  I* at = reinterpret_cast<I*>(t);
  K* kcopy = reinterpret_cast<K*>(t + ibytes);
  V* vcopy = reinterpret_cast<V*>(t + ibytes + kbytes);
  generic::parallel_for(stream_, n, iota_body<I>{at});
  stable_sort_tiles<I, no_value>(stream_, at, static_cast<no_value*>(nullptr), n, compare_at<I, K, Compare>{keys, comp});
  generic::parallel_for(stream_, n, gather_body<I, K>{keys, at, kcopy});
  throw_on_error(thrust_cdna4_memcpy_dtod(keys, kcopy, (std::size_t)n * sizeof(K), stream_), "merge sort: copy back");
  if (kHasValues) {
    generic::parallel_for(stream_, n, gather_body<I, V>{values, at, vcopy});
    throw_on_error(thrust_cdna4_memcpy_dtod(values, vcopy, (std::size_t)n * sizeof(V), stream_), "merge sort: copy back");
  }
}
template <class K, class V, class Compare>
void stable_sort_dispatch(void* stream_, K* keys, V* values, std::int64_t n, Compare comp, std::true_type /* tiles fit */) {
  stable_sort_tiles(stream_, keys, values, n, comp);
}
template <class K, class V, class Compare>
void stable_sort_dispatch(void* stream_, K* keys, V* values, std::int64_t n, Compare comp, std::false_type) {
  if (n <= 1) return;
  if (n <= (std::int64_t)0xFFFFFFFFll) stable_sort_positions<std::uint32_t>(stream_, keys, values, n, comp);
  else stable_sort_positions<std::uint64_t>(stream_, keys, values, n, comp);
}
template <class K, class V, class Compare>
void stable_sort(void* stream_, K* keys, V* values, std::int64_t n, Compare comp) {
  static_assert(thrust::detail::is_bytewise_movable<K>::value, "cdna4 merge sort: keys must be movable as bytes");
  static_assert(thrust::detail::is_bytewise_movable<V>::value, "cdna4 merge sort: values must be movable as bytes");
  stable_sort_dispatch(stream_, keys, values, n, comp, std::integral_constant<bool, tiles_fit_lds<K, V>()>());
}

template <class K, class V, class Compare>
void stable_sort_tiles(void* stream_, K* keys, V* values, std::int64_t n, Compare comp) {
  constexpr int IPT = items_per_thread<K, V>();
  constexpr int kTile = kBlock * IPT;
  constexpr bool kHasValues = !std::is_same<V, no_value>::value;
  static_assert((sizeof(K) + (kHasValues ? sizeof(V) : 0) + 2) * kTile <= 65536,
                "cdna4 merge sort: a tile of keys and values must fit the 64 KiB of static LDS");
  // the tile sort keeps two copies of keys and positions in LDS: its tiles are those of the merge
  // passes, or half of them where that is what fits
  constexpr int SORT_IPT = tile_sort_items<K, V, IPT>();
  constexpr int kSortTile = kBlock * SORT_IPT;
  if (n <= 1) return;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  const std::int64_t ntiles = (n + kTile - 1) / kTile;
  const std::int64_t nsorted = (n + kSortTile - 1) / kSortTile;

  hipLaunchKernelGGL((block_sort_kernel<SORT_IPT, K, V, Compare>), dim3((unsigned)nsorted), dim3(kBlock), 0, s, keys, values, n, comp);
  throw_on_error((int)hipGetLastError(), "merge sort: tile sort launch");
  if (nsorted == 1) return;

  const std::size_t kbytes = align256((std::size_t)n * sizeof(K));
  const std::size_t vbytes = kHasValues ? align256((std::size_t)n * sizeof(V)) : 0;
  const std::size_t sbytes = align256((std::size_t)(ntiles + 1) * sizeof(std::int64_t));
  temporary_storage tmp(kbytes + vbytes + sbytes, stream_);
  char* t = static_cast<char*>(tmp.data());
  K* kbuf[2] = {keys, reinterpret_cast<K*>(t)};
  V* vbuf[2] = {values, reinterpret_cast<V*>(t + kbytes)};
  std::int64_t* splits = reinterpret_cast<std::int64_t*>(t + kbytes + vbytes);

  int cur = 0;
  for (std::int64_t width = kSortTile; width < n; width *= 2) {
    hipLaunchKernelGGL((merge_partition_kernel<IPT, K, Compare>), dim3((unsigned)((ntiles + 255) / 256)), dim3(256), 0, s,
                       kbuf[cur], n, width, ntiles, splits, comp);
    hipLaunchKernelGGL((merge_kernel<IPT, K, V, Compare>), dim3((unsigned)ntiles), dim3(kBlock), 0, s, kbuf[cur], vbuf[cur],
                       kbuf[cur ^ 1], vbuf[cur ^ 1], n, width, ntiles, splits, comp);
    throw_on_error((int)hipGetLastError(), "merge sort: merge pass launch");
    cur ^= 1;
  }
  if (cur == 1) {  // odd number of passes: bring the result home
    throw_on_error(thrust_cdna4_memcpy_dtod(kbuf[0], kbuf[1], (std::size_t)n * sizeof(K), stream_), "merge sort: copy back");
    if (kHasValues)
      throw_on_error(thrust_cdna4_memcpy_dtod(vbuf[0], vbuf[1], (std::size_t)n * sizeof(V), stream_), "merge sort: copy back");
  }
  // the temporary buffer is returned to the pool in stream order when `tmp` goes out of scope
}

}}}}}  // namespace thrust::system::cdna4::detail::merge
