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
// A tile is 512 threads x ITEMS consecutive elements per thread (read and written in wavefront-
// contiguous pieces and reordered through LDS).  Tiles take their index from a
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

constexpr int kScanBlock = 512;
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

// An accumulator from `d` lanes below (undefined in lanes < d), word by word.
template <class Acc>
__device__ inline Acc shfl_up_acc(const Acc& a, int d) {
  constexpr int NW = (int)((sizeof(Acc) + 3) / 4);
  unsigned w[NW] = {};
  __builtin_memcpy(w, &a, sizeof(Acc));
#pragma unroll
  for (int k = 0; k < NW; k++) w[k] = __shfl_up(w[k], (unsigned)d, 64);
  Acc r;
  __builtin_memcpy(&r, w, sizeof(Acc));
  return r;
}

// Slot of element e of a tile in the staging buffer: one slot of padding after every ITEMS, so
// that both the striped order (consecutive lanes, consecutive elements) and the blocked order
// (consecutive lanes, ITEMS elements apart) spread over the LDS banks.
template <int ITEMS>
__device__ inline int staged(int e) { return e + e / ITEMS; }

// words[0, tiles * NW) are the descriptors, words[tiles * NW] is the ticket counter
template <class Op>
__global__ __launch_bounds__(kScanBlock) void scan_engine_kernel(std::int64_t n, Op op, unsigned long long* words, std::int64_t tiles) {
  typedef typename Op::acc Acc;
  typedef scan_desc<Acc> Desc;
  constexpr int ITEMS = scan_items(sizeof(Acc));
  constexpr int TILE = kScanBlock * ITEMS;
  constexpr int NWAVES = kScanBlock / 64;
  // Global memory is touched in striped order (thread t, step j: element j * 512 + t of the tile,
  // so a wavefront's access is one contiguous piece) while the scan wants every thread to own
  // ITEMS consecutive elements: loaded accumulators and results change order through LDS.
  // Accumulators too large for that buffer are loaded and stored in the threads' own order.
  constexpr bool kStaged = sizeof(Acc) * (TILE + TILE / ITEMS) <= 40 * 1024;
  typedef typename std::aligned_storage<sizeof(Acc), alignof(Acc)>::type Raw;
  __shared__ Raw raw_stage[kStaged ? TILE + TILE / ITEMS : 1], raw_wave[NWAVES], raw_look[64], raw_prefix;
  __shared__ unsigned long long s_tile;
  __shared__ int s_has_prefix;
  Acc* s_stage = reinterpret_cast<Acc*>(raw_stage);
  Acc* s_wave = reinterpret_cast<Acc*>(raw_wave);  // inclusive aggregate of each wavefront's threads
  Acc* s_look = reinterpret_cast<Acc*>(raw_look);  // one look-back window
  Acc* s_prefix = reinterpret_cast<Acc*>(&raw_prefix);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  if (tid == 0) s_tile = __hip_atomic_fetch_add(&words[tiles * Desc::NW], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const std::int64_t tile = (std::int64_t)s_tile;
  const std::int64_t tile_base = tile * TILE;
  const std::int64_t base = tile_base + (std::int64_t)tid * ITEMS;
  const std::int64_t left = n - base;
  const int count = left >= ITEMS ? ITEMS : left > 0 ? (int)left : 0;  // this thread's elements
  const std::int64_t tile_left = n - tile_base;                         // >= 1: tile < tiles
  const bool whole = tile_left >= TILE;
  const int nvalid = whole ? kScanBlock : (int)((tile_left + ITEMS - 1) / ITEMS);  // threads with elements
  const int tile_count = whole ? TILE : (int)tile_left;

  // every thread loads ITEMS times (the last element where the tile has no more) so that the
  // loads stay independent of each other
  Acc x[ITEMS];
  if constexpr (kStaged) {
    if (whole) {
#pragma unroll
      for (int j = 0; j < ITEMS; j++) x[j] = op.load(tile_base + j * kScanBlock + tid);
    } else {
#pragma unroll
      for (int j = 0; j < ITEMS; j++) {
        const std::int64_t i = tile_base + j * kScanBlock + tid;
        x[j] = op.load(i < n ? i : n - 1);
      }
    }
#pragma unroll
    for (int j = 0; j < ITEMS; j++) s_stage[staged<ITEMS>(j * kScanBlock + tid)] = x[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ITEMS; j++) x[j] = s_stage[staged<ITEMS>(tid * ITEMS + j)];
  } else {
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
      const std::int64_t i = base + j;
      x[j] = op.load(i < n ? i : n - 1);
    }
  }
  // inclusive scan of the thread's own elements (x is only ever indexed by unrolled constants, so
  // that it stays in registers)
  Acc incl = x[0];
#pragma unroll
  for (int j = 1; j < ITEMS; j++)
    if (j < count) {
      x[j] = op.combine(x[j - 1], x[j]);
      incl = x[j];
    }

  // inclusive scan of the threads' aggregates within each wavefront; threads without elements are
  // a suffix of the tile and stay out of it (no identity element is assumed)
  const bool valid = tid < nvalid;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const Acc up = shfl_up_acc(incl, d);
    if (valid && lane >= d) incl = op.combine(up, incl);
  }
  const Acc lane_before = shfl_up_acc(incl, 1);  // aggregate of the wavefront's earlier threads (lane > 0)
  const int last_valid = nvalid - 1;             // >= 0
  if (valid && (lane == 63 || tid == last_valid)) s_wave[wave] = incl;
  __syncthreads();
  const int nwaves_valid = (last_valid >> 6) + 1;

  if (wave == 0) {  // wavefront 0: publish, look back, publish again
    Acc tile_agg = s_wave[0];
    for (int w = 1; w < nwaves_valid; w++) tile_agg = op.combine(tile_agg, s_wave[w]);
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

  // everything before the thread's first element: tile prefix, earlier wavefronts, earlier lanes
  const bool tile_has = s_has_prefix != 0;
  bool thread_has = tile_has;
  Acc thread_before = x[0];  // placeholder until thread_has
  if (tile_has) thread_before = *s_prefix;
  for (int w = 0; w < wave; w++) {
    thread_before = thread_has ? op.combine(thread_before, s_wave[w]) : s_wave[w];
    thread_has = true;
  }
  if (lane > 0) {
    thread_before = thread_has ? op.combine(thread_before, lane_before) : lane_before;
    thread_has = true;
  }

  if constexpr (kStaged) {
    // results go to the staging buffer in the threads' order and leave it in striped order; the
    // value before element e is the result of element e - 1 (the tile's prefix for e = 0)
#pragma unroll
    for (int j = 0; j < ITEMS; j++)
      if (j < count) s_stage[staged<ITEMS>(tid * ITEMS + j)] = thread_has ? op.combine(thread_before, x[j]) : x[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
      const int e = j * kScanBlock + tid;
      if (e < tile_count) {
        const Acc upto = s_stage[staged<ITEMS>(e)];
        const bool has_before = e > 0 || tile_has;
        const Acc before = e > 0 ? s_stage[staged<ITEMS>(e - 1)] : (tile_has ? *s_prefix : upto);
        op.store(tile_base + e, has_before, before, upto);
      }
    }
  } else if (count > 0) {
    bool has_before = thread_has;
    Acc before = thread_before;
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
