// One-pass prefix engine with user functors and arbitrary accumulator types, as a kernel template:
// the path of inclusive_scan / exclusive_scan / *_scan_by_key / reduce_by_key for everything the
// precompiled kernels behind the C ABI do not cover (user-defined operators and predicates, an
// accumulator type that differs from the element type, struct elements).  The reference's kernels
// are generic in the same way: ScanOp, EqualityOp, ReductionOp and AccumT are template parameters of
// thrust/system/cuda/detail/scan.h:57-204, scan_by_key.h:69-282 and reduce_by_key.h:204-1058.
//
// An operation supplies
//     typedef ... acc;                                       trivially copyable accumulator
//     acc  load(int64 i) const;                              element i as an accumulator
//     acc  combine(const acc& a, const acc& b) const;        associative; a is the earlier range
//     void store(int64 i, bool has_before, const acc& before, const acc& upto) const;
// and the engine calls store(i, ...) once for every i in [0, n) with
//     before = load(0) (+) ... (+) load(i-1)   (meaningful when has_before, i.e. i > 0)
//     upto   = before (+) load(i).
// No identity element is needed and combine is never called with swapped arguments.
//
// A tile is 256 threads x ITEMS consecutive elements per thread.  Tiles take their index from a
// ticket counter, so every tile a waiting tile looks back at has started and the wait ends.  A
// tile descriptor is NW 64-bit atoms, one per 32-bit word of the accumulator, each (status << 32
// | word), written and read with relaxed agent-scope atomics: a reader that finds the same status
// in all NW atoms has a consistent value, so no fence is needed (each atom is written once per
// status).  One wavefront looks back 64 tiles at a time; because combine need not commute, the
// window is folded in tile order by one lane.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/cdna4/detail/scan_engine.h holds device kernel templates: compile with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <cstdint>
#include <type_traits>
#include <thrust/system/cdna4/detail/core.h>
#include <thrust/system/cdna4/detail/parallel_for.h>

namespace thrust { namespace system { namespace cdna4 { namespace detail { namespace generic {

constexpr int kScanBlock = 256;
constexpr unsigned kScanSpinLimit = 1u << 22;
constexpr int scan_items(std::size_t acc_bytes) { return acc_bytes <= 4 ? 16 : acc_bytes <= 8 ? 8 : acc_bytes <= 16 ? 4 : 2; }

template <class Acc>
struct scan_desc {
  static constexpr int NW = (int)((sizeof(Acc) + 3) / 4);
  __device__ static void store(unsigned long long* words, std::int64_t tile, unsigned status, const Acc& a) {
    unsigned w[NW] = {};
    __builtin_memcpy(w, &a, sizeof(Acc));
#pragma unroll
    for (int k = 0; k < NW; k++)
      __hip_atomic_store(&words[tile * NW + k], ((unsigned long long)status << 32) | w[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // the status (0 while the atoms disagree or are not written yet)
  __device__ static unsigned load(const unsigned long long* words, std::int64_t tile, Acc& a) {
    unsigned w[NW], st = 0;
    bool same = true;
#pragma unroll
    for (int k = 0; k < NW; k++) {
      const unsigned long long x = __hip_atomic_load(&words[tile * NW + k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      w[k] = (unsigned)x;
      const unsigned s = (unsigned)(x >> 32);
      if (k == 0) st = s;
      else same = same && s == st;
    }
    __builtin_memcpy(&a, w, sizeof(Acc));
    return same ? st : 0u;
  }
};

// words[0, tiles * NW) are the descriptors, words[tiles * NW] is the ticket counter
template <class Op>
__global__ __launch_bounds__(kScanBlock) void scan_engine_kernel(std::int64_t n, Op op, unsigned long long* words, std::int64_t tiles) {
  typedef typename Op::acc Acc;
  typedef scan_desc<Acc> Desc;
  constexpr int ITEMS = scan_items(sizeof(Acc));
  constexpr int TILE = kScanBlock * ITEMS;
  __shared__ typename std::aligned_storage<sizeof(Acc), alignof(Acc)>::type raw_agg[kScanBlock], raw_look[64], raw_prefix;
  __shared__ unsigned long long s_tile;
  __shared__ int s_has_prefix;
  Acc* s_agg = reinterpret_cast<Acc*>(raw_agg);    // inclusive aggregate of threads 0..t of the tile
  Acc* s_look = reinterpret_cast<Acc*>(raw_look);  // one look-back window
  Acc* s_prefix = reinterpret_cast<Acc*>(&raw_prefix);
  const int tid = threadIdx.x, lane = tid & 63;

  if (tid == 0) s_tile = __hip_atomic_fetch_add(&words[tiles * Desc::NW], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const std::int64_t tile = (std::int64_t)s_tile;
  const std::int64_t tile_base = tile * TILE;
  const std::int64_t base = tile_base + (std::int64_t)tid * ITEMS;
  const std::int64_t left = n - base;
  const int count = left >= ITEMS ? ITEMS : left > 0 ? (int)left : 0;  // this thread's elements
  const std::int64_t tile_left = n - tile_base;                         // >= 1: tile < tiles
  const int nvalid = tile_left >= TILE ? kScanBlock : (int)((tile_left + ITEMS - 1) / ITEMS);  // threads with elements

  // every thread loads (the last element where it has none of its own) so that the loads stay
  // independent of each other; then the inclusive scan of the thread's own elements
  Acc x[ITEMS];
  if (tile_left >= TILE) {
#pragma unroll
    for (int j = 0; j < ITEMS; j++) x[j] = op.load(base + j);
  } else {
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
      const std::int64_t i = base + j;
      x[j] = op.load(i < n ? i : n - 1);
    }
  }
#pragma unroll
  for (int j = 1; j < ITEMS; j++)
    if (j < count) x[j] = op.combine(x[j - 1], x[j]);

  // inclusive scan of the threads' aggregates through LDS; threads without elements are a suffix
  // of the tile and stay out of it
  if (count > 0) s_agg[tid] = x[count - 1];
  __syncthreads();
#pragma unroll
  for (int d = 1; d < kScanBlock; d <<= 1) {
    const bool take = tid >= d && tid < nvalid;
    Acc merged;
    if (take) merged = op.combine(s_agg[tid - d], s_agg[tid]);
    __syncthreads();
    if (take) s_agg[tid] = merged;
    __syncthreads();
  }

  if (tid < 64) {  // wavefront 0: publish, look back, publish again
    const Acc tile_agg = s_agg[nvalid - 1];
    bool has_prefix = false;  // meaningful in lane 0
    Acc prefix = tile_agg;    // placeholder until has_prefix
    if (tile > 0) {
      if (lane == 0) Desc::store(words, tile, 1u, tile_agg);
      std::int64_t nearest = tile - 1;
      unsigned spins = 0;
      for (;;) {
        const std::int64_t t = nearest - lane;  // lane 0 looks at the nearest tile before this one
        Acc val = tile_agg;
        unsigned status = 2u;  // before tile 0: an empty, fully known prefix
        if (t >= 0) status = Desc::load(words, t, val);
        const unsigned long long full = __builtin_amdgcn_ballot_w64(status == 2u);
        const unsigned long long empty = __builtin_amdgcn_ballot_w64(status == 0u);
        // lanes up to and including the nearest complete descriptor contribute
        const unsigned long long use = full ? ((full & (0ull - full)) << 1) - 1ull : ~0ull;
        // (the tiles waited for hold earlier tickets, so they are running and will publish; the
        // poll limit — seconds — only makes sure that this loop ends whatever happens)
        if ((empty & use) && ++spins < kScanSpinLimit) {
          __builtin_amdgcn_s_sleep(1);
          continue;
        }
        s_look[lane] = val;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (lane == 0) {
          const int last = full ? __builtin_ctzll(full) : 63;  // the farthest lane that counts
          bool has = false;
          Acc a = tile_agg;
          for (int l = last; l >= 0; l--) {  // in tile order: far to near
            if (nearest - l < 0) continue;   // the virtual tile before tile 0
            a = has ? op.combine(a, s_look[l]) : s_look[l];
            has = true;
          }
          if (has) {
            prefix = has_prefix ? op.combine(a, prefix) : a;
            has_prefix = true;
          }
        }
        __builtin_amdgcn_wave_barrier();
        if (full) break;
        nearest -= 64;
      }
    }
    if (lane == 0) {
      Desc::store(words, tile, 2u, has_prefix ? op.combine(prefix, tile_agg) : tile_agg);
      if (has_prefix) *s_prefix = prefix;
      s_has_prefix = has_prefix ? 1 : 0;
    }
  }
  __syncthreads();

  if (count > 0) {
    const bool tile_has = s_has_prefix != 0;
    bool has_before = tile_has || tid > 0;
    Acc before = x[0];  // placeholder until has_before
    if (tid > 0) before = tile_has ? op.combine(*s_prefix, s_agg[tid - 1]) : s_agg[tid - 1];
    else if (tile_has) before = *s_prefix;
    const Acc thread_before = before;
    const bool thread_has = has_before;
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
      if (j < count) {
        const Acc upto = thread_has ? op.combine(thread_before, x[j]) : x[j];
        op.store(base + j, has_before, before, upto);
        before = upto;
        has_before = true;
      }
    }
  }
}

template <class Op>
void scan_engine(void* stream_, std::int64_t n, Op op) {
  typedef typename Op::acc Acc;
  static_assert(std::is_trivially_copyable<Acc>::value, "cdna4 scan: the accumulator type must be trivially copyable");
  if (n <= 0) return;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  constexpr std::int64_t kTile = (std::int64_t)kScanBlock * scan_items(sizeof(Acc));
  const std::int64_t tiles = (n + kTile - 1) / kTile;
  const std::int64_t nwords = tiles * scan_desc<Acc>::NW + 1;
  temporary_storage tmp((std::size_t)nwords * sizeof(unsigned long long), stream_);
  unsigned long long* words = static_cast<unsigned long long*>(tmp.data());
  hipLaunchKernelGGL((select_init_kernel<unsigned long long>), dim3((unsigned)((nwords + 255) / 256)), dim3(256), 0, s, words, nwords);
  hipLaunchKernelGGL((scan_engine_kernel<Op>), dim3((unsigned)tiles), dim3(kScanBlock), 0, s, n, op, words, tiles);
  throw_on_error((int)hipGetLastError(), "scan: launch");
}

}}}}}  // namespace thrust::system::cdna4::detail::generic
