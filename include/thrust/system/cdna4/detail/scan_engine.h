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
// A tile is one or two parts of 512 threads x ITEMS consecutive elements per thread (read and
// written in wavefront-contiguous pieces and reordered through LDS).  Tiles take their index from a
// ticket counter, so every tile a waiting tile looks back at has started and the wait ends.  A
// tile descriptor is NW 64-bit atoms, one per 32-bit word of the accumulator, each (status << 32
// | word), written and read with relaxed agent-scope atomics: a reader that finds the same status
// in all NW atoms has a consistent value, so no fence is needed (each atom is written once per
// status).  One wavefront looks back 64 tiles at a time; because combine need not commute, the
// window is folded in tile order (a suffix reduction over the lanes).
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
    __builtin_memcpy(static_cast<void*>(&a), w, sizeof(Acc));
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
  __builtin_memcpy(static_cast<void*>(&r), w, sizeof(Acc));
  return r;
}

// An accumulator from `d` lanes above (undefined in lanes >= 64 - d), word by word.
template <class Acc>
__device__ inline Acc shfl_down_acc(const Acc& a, int d) {
  constexpr int NW = (int)((sizeof(Acc) + 3) / 4);
  unsigned w[NW] = {};
  __builtin_memcpy(w, &a, sizeof(Acc));
#pragma unroll
  for (int k = 0; k < NW; k++) w[k] = __shfl_down(w[k], (unsigned)d, 64);
  Acc r;
  __builtin_memcpy(static_cast<void*>(&r), w, sizeof(Acc));
  return r;
}

// Slot of element e of a tile in the staging buffer: one slot of padding after every ITEMS, so
// that both the striped order (consecutive lanes, consecutive elements) and the blocked order
// (consecutive lanes, ITEMS elements apart) spread over the LDS banks.
template <int ITEMS>
__device__ inline int staged(int e) { return e + e / ITEMS; }

// Parts of a tile: a tile is SUB parts of 512 x ITEMS elements each, staged through LDS one after
// the other, with ONE ticket, one descriptor and one look-back for all of them — the fixed costs
// of a tile are paid per SUB x 512 x ITEMS elements while LDS holds one part.
constexpr int scan_parts(std::size_t acc_bytes) { return acc_bytes <= 16 ? 2 : 1; }

// (has_a ? a : nothing) (+) (has_b ? b : nothing), for operators without an identity
template <class Op, class Acc>
__device__ inline void join(const Op& op, bool& has_a, Acc& a, bool has_b, const Acc& b) {
  if (has_b) {
    a = has_a ? op.combine(a, b) : b;
    has_a = true;
  }
}

// words[0, tiles * NW) are the descriptors, words[tiles * NW] is the ticket counter
template <class Op>
__global__ __launch_bounds__(kScanBlock) void scan_engine_kernel(std::int64_t n, Op op, unsigned long long* words, std::int64_t tiles, unsigned* timeouts) {
  typedef typename Op::acc Acc;
  typedef scan_desc<Acc> Desc;
  constexpr int ITEMS = scan_items(sizeof(Acc));
  constexpr int SUB = scan_parts(sizeof(Acc));
  constexpr int PART = kScanBlock * ITEMS;
  constexpr int TILE = SUB * PART;
  constexpr int NWAVES = kScanBlock / 64;
  // Global memory is touched in striped order (thread t, step j: element j * 512 + t of a part,
  // so a wavefront's access is one contiguous piece) while the scan wants every thread to own
  // ITEMS consecutive elements: loaded accumulators and results change order through LDS.
  // Accumulators too large for that buffer are loaded and stored in the threads' own order.
  constexpr bool kStaged = sizeof(Acc) * (PART + PART / ITEMS) <= 40 * 1024;
  typedef typename std::aligned_storage<sizeof(Acc), alignof(Acc)>::type Raw;
  __shared__ Raw raw_stage[kStaged ? PART + PART / ITEMS : 1], raw_wave[SUB][NWAVES], raw_part[SUB], raw_prefix;
  __shared__ unsigned long long s_tile;
  __shared__ int s_has_prefix;
  Acc* s_stage = reinterpret_cast<Acc*>(raw_stage);
  Acc* s_prefix = reinterpret_cast<Acc*>(&raw_prefix);
  const auto s_wave = [&](int part, int w) -> Acc& { return *reinterpret_cast<Acc*>(&raw_wave[part][w]); };  // inclusive aggregate of a wavefront's threads
  const auto s_part = [&](int part) -> Acc& { return *reinterpret_cast<Acc*>(&raw_part[part]); };           // aggregate of a part
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  if (tid == 0) s_tile = __hip_atomic_fetch_add(&words[tiles * Desc::NW], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const std::int64_t tile = (std::int64_t)s_tile;
  const std::int64_t tile_base = tile * TILE;
  const bool whole = n - tile_base >= TILE;  // every element of the tile exists (n - tile_base >= 1: tile < tiles)

  // elements of part p: how many exist, how many of them are this thread's, how many threads have any
  int part_count[SUB], count[SUB], nvalid[SUB];
#pragma unroll
  for (int p = 0; p < SUB; p++) {
    const std::int64_t left = n - (tile_base + (std::int64_t)p * PART);
    part_count[p] = whole ? PART : left >= PART ? PART : left > 0 ? (int)left : 0;
    const int mine = part_count[p] - tid * ITEMS;
    count[p] = mine >= ITEMS ? ITEMS : mine > 0 ? mine : 0;
    nvalid[p] = (part_count[p] + ITEMS - 1) / ITEMS;
  }

  // every thread loads SUB x ITEMS times (the last element where the input has no more) so that
  // the loads stay independent of each other
  Acc x[SUB][ITEMS];
#pragma unroll
  for (int p = 0; p < SUB; p++) {
    const std::int64_t part_base = tile_base + (std::int64_t)p * PART;
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
      const std::int64_t i = part_base + (kStaged ? j * kScanBlock + tid : tid * ITEMS + j);
      x[p][j] = op.load(whole ? i : (i < n ? i : n - 1));
    }
  }

  Acc lane_before[SUB];  // aggregate of the wavefront's earlier threads in part p (lane > 0)
#pragma unroll
  for (int p = 0; p < SUB; p++) {
    if constexpr (kStaged) {
      if (p > 0) __syncthreads();  // the part before has been read out of the buffer
#pragma unroll
      for (int j = 0; j < ITEMS; j++) s_stage[staged<ITEMS>(j * kScanBlock + tid)] = x[p][j];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < ITEMS; j++) x[p][j] = s_stage[staged<ITEMS>(tid * ITEMS + j)];
    }
    // inclusive scan of the thread's own elements (x is only ever indexed by unrolled constants,
    // so that it stays in registers)
    Acc incl = x[p][0];
#pragma unroll
    for (int j = 1; j < ITEMS; j++)
      if (j < count[p]) {
        x[p][j] = op.combine(x[p][j - 1], x[p][j]);
        incl = x[p][j];
      }
    // inclusive scan of the threads' aggregates within each wavefront; threads without elements
    // are a suffix of the part and stay out of it (no identity element is assumed)
    const bool valid = tid < nvalid[p];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const Acc up = shfl_up_acc(incl, d);
      if (valid && lane >= d) incl = op.combine(up, incl);
    }
    lane_before[p] = shfl_up_acc(incl, 1);
    if (valid && (lane == 63 || tid == nvalid[p] - 1)) s_wave(p, wave) = incl;
  }
  __syncthreads();

  if (wave == 0) {  // wavefront 0: aggregates of the parts and of the tile, publish, look back, publish again
    bool has_agg = false;
    Acc tile_agg = x[0][0];  // placeholder until has_agg (part 0 is never empty)
#pragma unroll
    for (int p = 0; p < SUB; p++) {
      const int nw = (nvalid[p] + 63) >> 6;  // wavefronts with elements in part p
      bool has = false;
      Acc agg = tile_agg;
      for (int w = 0; w < nw; w++) join(op, has, agg, true, s_wave(p, w));
      if (has && lane == 0) s_part(p) = agg;
      join(op, has_agg, tile_agg, has, agg);
    }
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
        if (empty & use) {
          if (++spins < kScanSpinLimit) {
            __builtin_amdgcn_s_sleep(1);
            continue;
          }
          // gives up and carries on with what it has; counted where the sort's time-outs are
          // (thrust_cdna4_lookback_timeouts)
          if (lane == 0 && timeouts) atomicAdd(timeouts, 1u);
        }
        // The window is folded in tile order — far to near, combine need not commute — by a
        // suffix reduction over the lanes: after step d lane l holds lanes l + 2d - 1 ... l.
        // Lanes beyond the nearest complete descriptor, and the virtual tiles before tile 0, stay out.
        int last = full ? __builtin_ctzll(full) : 63;  // the farthest lane that counts
        if ((std::int64_t)last > nearest) last = (int)nearest;
        Acc a = val;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const Acc farther = shfl_down_acc(a, d);
          if (lane + d <= last) a = op.combine(farther, a);
        }
        if (lane == 0 && last >= 0) {
          prefix = has_prefix ? op.combine(a, prefix) : a;
          has_prefix = true;
        }
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

  // everything before part p: the tile's prefix and the parts before it
  bool part_has = s_has_prefix != 0;
  Acc part_before = x[0][0];  // placeholder until part_has
  if (part_has) part_before = *s_prefix;
#pragma unroll
  for (int p = 0; p < SUB; p++) {
    if (part_count[p] > 0) {
      // everything before the thread's first element of the part: earlier wavefronts, earlier lanes
      bool thread_has = part_has;
      Acc thread_before = part_before;
      if (count[p] > 0) {  // (a thread without elements has no use for it, and the wavefronts before it may have none either)
        for (int w = 0; w < wave; w++) join(op, thread_has, thread_before, true, s_wave(p, w));
        join(op, thread_has, thread_before, lane > 0, lane_before[p]);
      }
      const std::int64_t part_base = tile_base + (std::int64_t)p * PART;
      if constexpr (kStaged) {
        // results go to the staging buffer in the threads' order and leave it in striped order;
        // the value before element e is the result of element e - 1 (the part's prefix for e = 0)
        __syncthreads();  // the buffer is free: the loads of the last part, or the stores of the part before, are done
#pragma unroll
        for (int j = 0; j < ITEMS; j++)
          if (j < count[p]) s_stage[staged<ITEMS>(tid * ITEMS + j)] = thread_has ? op.combine(thread_before, x[p][j]) : x[p][j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
          const int e = j * kScanBlock + tid;
          if (e < part_count[p]) {
            const Acc upto = s_stage[staged<ITEMS>(e)];
            const bool has_before = e > 0 || part_has;
            const Acc before = e > 0 ? s_stage[staged<ITEMS>(e - 1)] : (part_has ? part_before : upto);
            op.store(part_base + e, has_before, before, upto);
          }
        }
      } else if (count[p] > 0) {
        bool has_before = thread_has;
        Acc before = thread_before;
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
          if (j < count[p]) {
            const Acc upto = thread_has ? op.combine(thread_before, x[p][j]) : x[p][j];
            op.store(part_base + tid * ITEMS + j, has_before, before, upto);
            before = upto;
            has_before = true;
          }
        }
      }
      if (p + 1 < SUB) join(op, part_has, part_before, true, s_part(p));
    }
  }
}

template <class Op>
void scan_engine(void* stream_, std::int64_t n, Op op) {
  typedef typename Op::acc Acc;
  static_assert(thrust::detail::is_bytewise_movable<Acc>::value, "cdna4 scan: the accumulator type must be movable as bytes");
  if (n <= 0) return;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  constexpr std::int64_t kTile = (std::int64_t)kScanBlock * scan_items(sizeof(Acc)) * scan_parts(sizeof(Acc));
  const std::int64_t tiles = (n + kTile - 1) / kTile;
  const std::int64_t nwords = tiles * scan_desc<Acc>::NW + 1;
  temporary_storage tmp((std::size_t)nwords * sizeof(unsigned long long), stream_);
  unsigned long long* words = static_cast<unsigned long long*>(tmp.data());
  hipLaunchKernelGGL((select_init_kernel<unsigned long long>), dim3((unsigned)((nwords + 255) / 256)), dim3(256), 0, s, words, nwords);
  void* timeouts = nullptr;  // the library's per-device counter of waits that did not end
  throw_on_error(thrust_cdna4_lookback_timeout_counter(&timeouts), "scan: time-out counter");
  hipLaunchKernelGGL((scan_engine_kernel<Op>), dim3((unsigned)tiles), dim3(kScanBlock), 0, s, n, op, words, tiles,
                     static_cast<unsigned*>(timeouts));
  throw_on_error((int)hipGetLastError(), "scan: launch");
}

}}}}}  // namespace thrust::system::cdna4::detail::generic
