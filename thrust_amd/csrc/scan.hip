// Single-pass prefix scan with decoupled look-back for gfx950.
//
// One launch reads every element once and writes it once.  A workgroup takes a tile by
// atomic ticket, loads it with 128-bit accesses (thread t owns 16 bytes of every 16·BLOCK
// byte chunk, so loads and stores of a wave are contiguous), scans it with DPP wave scans,
// publishes the tile aggregate, obtains the prefix of all earlier tiles by look-back and
// writes the result.  Semantics: thrust/system/detail/sequential/scan.h:47-114; replaces
// thrust/system/cuda/detail/scan.h:57-204 (cub::DispatchScan).
#include <mutex>

#include "common.h"

namespace tcd {

template <class T>
struct alignas(16) Vec16 {
  T v[16 / sizeof(T)];
};

// TICKET: tiles are handed out by an atomic counter, so every tile a tile waits on has started
// (used when the output overlaps the input).  Otherwise a tile is the workgroup of the same
// index — no atomic and no barrier before the loads, 6 % faster at 2^28 and 25 % at 2^24 — and a
// descriptor that stays missing is recomputed from the input after `patience` polls.
// minimum(a, b) = a < b ? a : b over floating-point values with NaNs: the serial fold RESTARTS at
// every NaN (acc < NaN is false, so the NaN replaces the accumulator; NaN < x is false too, so the
// next element replaces the NaN).  What a piece of the input contributes to a fold is then a pair:
// the raw fold of the piece, and whether the piece holds a NaN — in which case nothing to its left
// survives it.  Pairs combine associatively, so they travel through the wavefront scans and the
// tile descriptors in place of the plain value.  Only the floating-point minimum instantiations
// carry them.
template <class T, class Op>
struct scan_restarts {
  static constexpr bool value = std::is_floating_point<T>::value && std::is_same<Op, OpMinimum>::value;
};
template <class T>
struct RestartPair {
  uint32_t a[sizeof(T) / 4];  // the value's words (keeps an 8-byte value from padding the pair to 16 bytes)
  uint32_t r;                 // 0: the piece holds no NaN, 1: it does, 2: the piece is empty
  __device__ T value() const { T v; __builtin_memcpy(&v, a, sizeof(T)); return v; }
  __device__ static RestartPair make(T v, uint32_t r) {
    RestartPair p;
    __builtin_memcpy(p.a, &v, sizeof(T));
    p.r = r;
    return p;
  }
  // The empty piece has a state of its own because the operator's identity is none for a NaN:
  // minimum(NaN, +inf) is +inf, and an exclusive scan shows the accumulator itself.
  template <class Op>
  __device__ static RestartPair combine(const RestartPair& x, const RestartPair& y) {
    if (y.r == 2u) return x;
    if (x.r == 2u) return y;
    return make(y.r ? y.value() : Op::template apply<T>(x.value(), y.value()), x.r | y.r);
  }
};
// what a tile publishes and what travels across lanes: a dword container for 1- and 2-byte T
template <class T, class Op>
struct scan_payload {
  using type = typename std::conditional<scan_restarts<T, Op>::value, RestartPair<T>,
                                         typename std::conditional<(sizeof(T) < 4), uint32_t, T>::type>::type;
};

template <class T, class Op, int BLOCK, int CHUNKS, bool TICKET>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4))) void scan_kernel(const T* in, T* out, int64_t n, T init,
                                                     int exclusive, uint64_t* desc,
                                                     uint32_t* ticket, int vec_ok, int patience, int publish_delay) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NWAVES = BLOCK / kWave;
  constexpr int64_t TILE = (int64_t)BLOCK * VEC * CHUNKS;
  // cross-lane traffic, LDS and descriptors carry W
  using W = typename scan_payload<T, Op>::type;
  constexpr bool kRestarts = scan_restarts<T, Op>::value;
  static_assert(!kRestarts || TICKET, "pieces of a restarting fold combine in input order only: no recomputation from strided reads");

  __shared__ W s_tot[CHUNKS * NWAVES];  // inclusive total of (chunk, wave), then its exclusive offset
  __shared__ uint32_t s_tile;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const T id = Op::template identity<T>();
  auto op = [](T a, T b) { return Op::template apply<T>(a, b); };
  auto toW = [](T a) {
    if constexpr (kRestarts) return W::make(a, __builtin_isnan(a) ? 1u : 0u);
    else if constexpr (std::is_same<W, T>::value) return a;
    else return (W)(typename unsigned_of<T>::type)a;
  };
  auto fromW = [](const W& w) {
    if constexpr (kRestarts) return w.value();
    else return (T)w;
  };
  auto opW = [&](const W& a, const W& b) {
    if constexpr (kRestarts) return W::template combine<Op>(a, b);
    else if constexpr (std::is_same<W, T>::value) return op(a, b);
    else return (W)(typename unsigned_of<T>::type)op((T)a, (T)b);
  };
  W idW;
  if constexpr (kRestarts) idW = W::make(id, 2u);
  else idW = toW(id);

  int64_t tile = blockIdx.x;
  if constexpr (TICKET) {
    if (tid == 0) s_tile = atomicAdd(ticket, 1u);
    __syncthreads();
    tile = s_tile;
  }
  const int64_t base = tile * TILE;
  const bool fast = vec_ok && (base + TILE <= n);  // whole tile present, pointers aligned to their elements
  const T* tin = in + base + (int64_t)tid * VEC;
  T* tout = out + base + (int64_t)tid * VEC;

  // maximum(a, b) = a < b ? b : a over floating-point values with NaNs is not associative: the
  // serial fold keeps a NaN that STARTS it (NaN < x is false) and skips a NaN met later
  // (acc < NaN is false too).  So every NaN is replaced by the identity as it is loaded, which
  // leaves an associative fold, and the one NaN that the serial fold would have kept — the first
  // value of the fold: element 0, or `init` of an exclusive scan — is handled apart: all results
  // are then that NaN.  (An in-place scan may already have overwritten element 0: with the same
  // bits.)  Nothing of this is compiled for other types and operators.
  constexpr bool kNanAware = std::is_floating_point<T>::value && std::is_same<Op, OpMaximum>::value;
  T lead = id;
  if constexpr (kNanAware) lead = exclusive ? init : in[0];

  T x[CHUNKS][VEC];
  if (fast) {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      const Vec16<T> v = load16<Vec16<T>>(tin + c * BLOCK * VEC);
#pragma unroll
      for (int j = 0; j < VEC; j++) x[c][j] = v.v[j];
    }
  } else {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        const int64_t idx = base + ((int64_t)c * BLOCK + tid) * VEC + j;
        const T got = in[idx < n ? idx : n - 1];  // unconditional: a load under a branch waits for the one before
        x[c][j] = idx < n ? got : id;
      }
    }
  }
  if constexpr (kNanAware) {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++)
#pragma unroll
      for (int j = 0; j < VEC; j++) x[c][j] = __builtin_isnan(x[c][j]) ? id : x[c][j];
  }

  // thread-local inclusive scan of each 16-byte group, then a wave scan of the group sums
  T excl[CHUNKS];
  uint32_t nan_below = 0;  // kRestarts: bit c: a NaN in the wavefront's groups of chunk c below this thread's
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    if constexpr (kRestarts) {
      // the elements stay as loaded: the results are formed by one more raw fold from the
      // accumulator before the group, which restarts at NaNs by itself
      T acc = x[c][0];
      bool seen = __builtin_isnan(acc);
#pragma unroll
      for (int j = 1; j < VEC; j++) {
        seen = seen || __builtin_isnan(x[c][j]);
        acc = op(acc, x[c][j]);
      }
      const W incl = wave_inclusive_scan(W::make(acc, seen ? 1u : 0u), idW, opW);
      const W below = wave_shift_up1(incl, idW);  // empty in lane 0
      excl[c] = below.value();
      nan_below |= (below.r == 1u ? 1u : 0u) << c;
      if (lane == kWave - 1) s_tot[c * NWAVES + wave] = incl;
    } else {
#pragma unroll
      for (int j = 1; j < VEC; j++) x[c][j] = op(x[c][j - 1], x[c][j]);
      const W incl = wave_inclusive_scan(toW(x[c][VEC - 1]), idW, opW);
      excl[c] = fromW(wave_shift_up1(incl, idW));
      if (lane == kWave - 1) s_tot[c * NWAVES + wave] = incl;
    }
  }
  __syncthreads();

  // wave 0: exclusive scan of the (chunk, wave) totals in tile order (PER consecutive totals per
  // lane), then the look-back
  if (wave == 0) {
    constexpr int NTOT = CHUNKS * NWAVES;
    constexpr int PER = (NTOT + kWave - 1) / kWave;
    W mine[PER];
#pragma unroll
    for (int q = 0; q < PER; q++) {
      const int idx = lane * PER + q;
      mine[q] = idx < NTOT ? s_tot[idx] : idW;
      if (q > 0) mine[q] = opW(mine[q - 1], mine[q]);
    }
    const W incl = wave_inclusive_scan(mine[PER - 1], idW, opW);
    const W tile_agg = readlane(incl, kWave - 1);
    const W before = wave_shift_up1(incl, idW);  // totals of the lanes below
    // Descriptors carry sums of INPUT elements only.  `init` of an exclusive scan is applied by
    // every tile to its own prefix below, so a tile aggregate recomputed from the input by a
    // later tile (wave_lookback_or_compute) is the same value its owner would have published.
    W prefix = idW;
    if (tile == 0) {
      for (int i = 0; i < publish_delay; i++) __builtin_amdgcn_s_sleep(127);  // test knob, 0 in normal use
      if (lane == 0) TileDesc<W>::store(desc, 0, kInclusive, tile_agg);
    } else {
      if (lane == 0) TileDesc<W>::store(desc, tile, kPartial, tile_agg);
      if constexpr (TICKET) {
        prefix = wave_lookback<W>(desc, tile, idW, opW);
      } else {
        // the aggregate of an earlier tile (always a whole one), straight from the input
        // (a lane folds every 64th element: the operator must commute.  Floating-point maximum
        // does not where +0 meets -0 — the fold keeps the one that comes first — so there a lane
        // folds a contiguous piece and the pieces combine in lane order.)
        const auto aggregate_of = [&](int64_t t) -> W {
          constexpr int PIECE = (int)(TILE / kWave);
          constexpr int64_t STRIDE = kNanAware ? 1 : kWave;
          const T* p = in + t * TILE + (kNanAware ? (int64_t)lane * PIECE : (int64_t)lane);
          const auto element = [&](int k) {
            const T e = p[(int64_t)k * STRIDE];
            if constexpr (kNanAware) return __builtin_isnan(e) ? id : e;
            else return e;
          };
          T acc = element(0);
          if constexpr (kNanAware) {
#pragma unroll 2
            for (int k = 1; k < PIECE; k++) acc = op(acc, element(k));
          } else {
#pragma unroll 8
            for (int k = 1; k < PIECE; k++) acc = op(acc, element(k));
          }
          return readlane(wave_inclusive_scan(toW(acc), idW, opW), kWave - 1);
        };
        prefix = wave_lookback_or_compute<W>(desc, tile, idW, opW, patience, aggregate_of);
      }
      if (lane == 0) TileDesc<W>::store(desc, tile, kInclusive, opW(prefix, tile_agg));
    }
    if (exclusive) prefix = opW(toW(init), prefix);
    const W base_w = opW(prefix, before);
    // offset of (chunk, wave) in the whole input = everything before it
#pragma unroll
    for (int q = 0; q < PER; q++) {
      const int idx = lane * PER + q;
      if (idx < NTOT) s_tot[idx] = q == 0 ? base_w : opW(base_w, mine[q - 1]);
    }
  }
  __syncthreads();

  // results: element (c, j) = offset of its (chunk, wave) (+) lanes before it (+) its group prefix
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    if constexpr (kRestarts) {
      // the accumulator before the group: what lies before the wavefront's groups counts unless
      // those groups hold a NaN
      const T before_wave = fromW(s_tot[c * NWAVES + wave]);
      T acc = lane == 0 ? before_wave : ((nan_below >> c) & 1u) ? excl[c] : op(before_wave, excl[c]);
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        const T e = x[c][j];
        if (exclusive) x[c][j] = acc;
        acc = op(acc, e);
        if (!exclusive) x[c][j] = acc;
      }
    } else {
      const T off = op(fromW(s_tot[c * NWAVES + wave]), excl[c]);
      if (exclusive) {
#pragma unroll
        for (int j = VEC - 1; j > 0; j--) x[c][j] = op(off, x[c][j - 1]);
        x[c][0] = off;
      } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) x[c][j] = op(off, x[c][j]);
      }
    }
  }
  if constexpr (kNanAware) {
    if (__builtin_isnan(lead)) {
#pragma unroll
      for (int c = 0; c < CHUNKS; c++)
#pragma unroll
        for (int j = 0; j < VEC; j++) x[c][j] = lead;
    }
  }
  if (fast) {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      Vec16<T> v;
#pragma unroll
      for (int j = 0; j < VEC; j++) v.v[j] = x[c][j];
      store16(tout + c * BLOCK * VEC, v);
    }
  } else {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        const int64_t idx = base + ((int64_t)c * BLOCK + tid) * VEC + j;
        if (idx < n) out[idx] = x[c][j];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// The same scan for 1- and 2-byte elements.  Above, every element has a register of its own,
// which holds narrow types to 64 elements per thread and a tile to 32 KiB: too little per ticket
// and look-back.  Here the tile stays PACKED in registers (4 dwords per 16-byte chunk, 16 chunks
// per thread: 256 bytes, as for the wide types); an element is unpacked where it is used — once
// for the totals, once more when the results are formed and packed for the store.  The arithmetic
// is a few operations per element and far below the memory time.
// ---------------------------------------------------------------------------------------
template <class T>
__device__ inline T packed_get(const uint32_t (&r)[4], int j) {  // j is a constant after unrolling
  constexpr int PER = 4 / (int)sizeof(T);
  using U = typename unsigned_of<T>::type;
  return (T)(U)(r[j / PER] >> ((j % PER) * 8 * (int)sizeof(T)));
}
template <class T>
__device__ inline void packed_put(uint32_t (&r)[4], int j, T v) {
  constexpr int PER = 4 / (int)sizeof(T);
  using U = typename unsigned_of<T>::type;
  const uint32_t w = (uint32_t)(U)v << ((j % PER) * 8 * (int)sizeof(T));
  r[j / PER] = (j % PER) == 0 ? w : (r[j / PER] | w);
}

template <class T, class Op, int BLOCK, int CHUNKS, bool TICKET>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4))) void scan_packed_kernel(const T* in, T* out, int64_t n, T init,
                                                     int exclusive, uint64_t* desc,
                                                     uint32_t* ticket, int vec_ok, int patience, int publish_delay) {
  static_assert(sizeof(T) < 4, "1- and 2-byte elements");
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NWAVES = BLOCK / kWave;
  constexpr int64_t TILE = (int64_t)BLOCK * VEC * CHUNKS;
  using W = uint32_t;  // cross-lane traffic, LDS and descriptors carry a dword container
  using U = typename unsigned_of<T>::type;

  __shared__ W s_tot[CHUNKS * NWAVES];  // inclusive total of (chunk, wave), then its exclusive offset
  __shared__ uint32_t s_tile;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const T id = Op::template identity<T>();
  auto op = [](T a, T b) { return Op::template apply<T>(a, b); };
  auto toW = [](T a) { return (W)(U)a; };
  auto opW = [&](W a, W b) { return (W)(U)op((T)a, (T)b); };
  const W idW = toW(id);

  int64_t tile = blockIdx.x;
  if constexpr (TICKET) {
    if (tid == 0) s_tile = atomicAdd(ticket, 1u);
    __syncthreads();
    tile = s_tile;
  }
  const int64_t base = tile * TILE;
  // 128-bit accesses need no alignment here, so only the tile that the input ends in is special
  (void)vec_ok;
  const bool fast = base + TILE <= n;
  const T* tin = in + base + (int64_t)tid * VEC;
  T* tout = out + base + (int64_t)tid * VEC;

  // The chunk that the input ends in is put together element by element (a loop with a computed
  // shift, not unrolled: it runs once per call); chunks past the end hold the identity.
  const uint32_t id_word = (uint32_t)(U)id * (sizeof(T) == 1 ? 0x01010101u : 0x00010001u);
  auto load_tail = [&](const T* p, int count) {
    uint64_t half[2] = {((uint64_t)id_word << 32) | id_word, ((uint64_t)id_word << 32) | id_word};
#pragma unroll 1
    for (int j = 0; j < count; j++) {
      const int bit = j * 8 * (int)sizeof(T);
      const uint64_t mask = (uint64_t)(U)~U(0) << (bit & 63);
      const uint64_t e = (uint64_t)(U)p[j] << (bit & 63);
      if (bit < 64) half[0] = (half[0] & ~mask) | e;
      else half[1] = (half[1] & ~mask) | e;
    }
    tcd_v4u v;
    v.x = (uint32_t)half[0]; v.y = (uint32_t)(half[0] >> 32); v.z = (uint32_t)half[1]; v.w = (uint32_t)(half[1] >> 32);
    return v;
  };
  uint32_t x[CHUNKS][4];
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    tcd_v4u v;
    if (fast) {
      v = load16<tcd_v4u>(tin + c * BLOCK * VEC);
    } else {
      const int64_t left = n - (base + ((int64_t)c * BLOCK + tid) * VEC);  // elements from this chunk's first to the end
      v.x = v.y = v.z = v.w = id_word;
      if (left >= VEC) v = load16<tcd_v4u>(tin + c * BLOCK * VEC);
      else if (left > 0) v = load_tail(tin + c * BLOCK * VEC, (int)left);
    }
    x[c][0] = v.x; x[c][1] = v.y; x[c][2] = v.z; x[c][3] = v.w;
  }

  // total of each 16-byte group, then a wave scan of the group totals
  T excl[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    T acc = packed_get<T>(x[c], 0);
#pragma unroll
    for (int j = 1; j < VEC; j++) acc = op(acc, packed_get<T>(x[c], j));
    const W incl = wave_inclusive_scan(toW(acc), idW, opW);
    excl[c] = (T)wave_shift_up1(incl, idW);
    if (lane == kWave - 1) s_tot[c * NWAVES + wave] = incl;
  }
  __syncthreads();

  // wave 0: exclusive scan of the (chunk, wave) totals in tile order, then the look-back
  if (wave == 0) {
    constexpr int NTOT = CHUNKS * NWAVES;
    constexpr int PER = (NTOT + kWave - 1) / kWave;
    W mine[PER];
#pragma unroll
    for (int q = 0; q < PER; q++) {
      const int idx = lane * PER + q;
      mine[q] = idx < NTOT ? s_tot[idx] : idW;
      if (q > 0) mine[q] = opW(mine[q - 1], mine[q]);
    }
    const W incl = wave_inclusive_scan(mine[PER - 1], idW, opW);
    const W tile_agg = readlane(incl, kWave - 1);
    const W before = wave_shift_up1(incl, idW);  // totals of the lanes below
    // descriptors carry sums of INPUT elements only; `init` is applied by every tile to its own prefix
    W prefix = idW;
    if (tile == 0) {
      for (int i = 0; i < publish_delay; i++) __builtin_amdgcn_s_sleep(127);  // test knob, 0 in normal use
      if (lane == 0) TileDesc<W>::store(desc, 0, kInclusive, tile_agg);
    } else {
      if (lane == 0) TileDesc<W>::store(desc, tile, kPartial, tile_agg);
      if constexpr (TICKET) {
        prefix = wave_lookback<W>(desc, tile, idW, opW);
      } else {
        // the aggregate of an earlier tile (always a whole one), straight from the input
        const auto aggregate_of = [&](int64_t t) -> W {
          const T* p = in + t * TILE + lane;
          T acc = p[0];
#pragma unroll 8
          for (int k = 1; k < (int)(TILE / kWave); k++) acc = op(acc, p[(int64_t)k * kWave]);
          return readlane(wave_inclusive_scan(toW(acc), idW, opW), kWave - 1);
        };
        prefix = wave_lookback_or_compute<W>(desc, tile, idW, opW, patience, aggregate_of);
      }
      if (lane == 0) TileDesc<W>::store(desc, tile, kInclusive, opW(prefix, tile_agg));
    }
    if (exclusive) prefix = opW(toW(init), prefix);
    const W base_w = opW(prefix, before);
#pragma unroll
    for (int q = 0; q < PER; q++) {
      const int idx = lane * PER + q;
      if (idx < NTOT) s_tot[idx] = q == 0 ? base_w : opW(base_w, mine[q - 1]);
    }
  }
  __syncthreads();

  // results: the running value starts at the offset of the element's group and walks the group.
  // (The packed words pass through an empty asm first: the elements are unpacked again here, not
  // kept in registers of their own since the totals were formed.)
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    T run = op((T)s_tot[c * NWAVES + wave], excl[c]);
    uint32_t src[4], r[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      src[q] = x[c][q];
      asm volatile("" : "+v"(src[q]));
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      const T e = packed_get<T>(src, j);
      if (exclusive) {
        packed_put<T>(r, j, run);
        run = op(run, e);
      } else {
        run = op(run, e);
        packed_put<T>(r, j, run);
      }
    }
    tcd_v4u v;
    v.x = r[0]; v.y = r[1]; v.z = r[2]; v.w = r[3];
    if (fast) {
      store16(tout + c * BLOCK * VEC, v);
    } else {
      const int64_t left = n - (base + ((int64_t)c * BLOCK + tid) * VEC);
      if (left >= VEC) {
        store16(tout + c * BLOCK * VEC, v);
      } else if (left > 0) {
        const uint64_t half[2] = {((uint64_t)r[1] << 32) | r[0], ((uint64_t)r[3] << 32) | r[2]};
        T* p = tout + c * BLOCK * VEC;
#pragma unroll 1
        for (int j = 0; j < (int)left; j++) {
          const int bit = j * 8 * (int)sizeof(T);
          p[j] = (T)(U)((bit < 64 ? half[0] : half[1]) >> (bit & 63));
        }
      }
    }
  }
}

template <class T>
struct ScanConfig {
  // 256 bytes per thread (128 KiB tiles: fewer tickets and look-backs per byte; measured best on
  // MI355X: 64 KiB tiles are 10 % slower, 192 KiB tiles 3 %); 1- and 2-byte elements stay packed
  // in their registers (scan_packed_kernel).
  static constexpr int BLOCK = 512;
  static constexpr int CHUNKS = 16;
  static constexpr int64_t TILE = (int64_t)BLOCK * (16 / sizeof(T)) * CHUNKS;
};

template <class T, class Op>
static hipError_t scan_typed(void* temp, size_t* temp_bytes, int exclusive, const void* in,
                             void* out, int64_t n, const void* init, hipStream_t stream) {
  using C = ScanConfig<T>;
  using Payload = typename scan_payload<T, Op>::type;
  constexpr bool kRestarts = scan_restarts<T, Op>::value;
  const int64_t ntiles = ceil_div(n, C::TILE);
  const size_t need = 256 + align_up((size_t)ntiles * TileDesc<Payload>::kBytesPerTile, 256);
  if (temp == nullptr) {
    *temp_bytes = need;
    return hipSuccess;
  }
  if (*temp_bytes < need) return hipErrorInvalidValue;
  if (n == 0) return hipSuccess;
  // One tile consults no descriptor and reads its whole input before it writes any output: it
  // needs neither the cleared descriptors (a launch less: a third of a small call) nor tickets.
  // (the restarting fold of floating-point minimum always takes tickets: its kernel exists in
  // that form only)
  const bool single = ntiles == 1 && !kRestarts;
  if (!single) {
    const hipError_t e = zero_async(temp, need, stream);
    if (e != hipSuccess) return e;
  }
  T iv = T(0);
  if (init) __builtin_memcpy(&iv, init, sizeof(T));
  uint32_t* ticket = reinterpret_cast<uint32_t*>(temp);
  uint64_t* desc = reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256);
  // 128-bit accesses need no more than the elements' own alignment (see load16)
  const int vec_ok = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & (sizeof(T) - 1)) == 0;
  const bool ticketed = kRestarts || (!single && ranges_overlap(in, (size_t)n * sizeof(T), out, (size_t)n * sizeof(T)));
  const int patience = ticketed ? 0 : lookback_patience(), delay = ticketed ? 0 : lookback_test_publish_delay();
  auto launch = [&](auto kernel) {
    TCD_LAUNCH("scan_kernel", kernel, dim3((unsigned)ntiles), dim3(C::BLOCK), stream, static_cast<const T*>(in),
               static_cast<T*>(out), n, iv, exclusive, desc, ticket, vec_ok, patience, delay);
  };
  if constexpr (sizeof(T) < 4) {
    if (ticketed) launch(scan_packed_kernel<T, Op, C::BLOCK, C::CHUNKS, true>);
    else launch(scan_packed_kernel<T, Op, C::BLOCK, C::CHUNKS, false>);
  } else if constexpr (kRestarts) {
    launch(scan_kernel<T, Op, C::BLOCK, C::CHUNKS, true>);
  } else {
    if (ticketed) launch(scan_kernel<T, Op, C::BLOCK, C::CHUNKS, true>);
    else launch(scan_kernel<T, Op, C::BLOCK, C::CHUNKS, false>);
  }
  return hipGetLastError();
}

}  // namespace tcd

extern "C" int thrust_cdna4_scan(void* temp, size_t* temp_bytes, int dtype, int op, int exclusive,
                                 const void* in, void* out, int64_t n, const void* init,
                                 void* stream) {
  using namespace tcd;
  if (!temp_bytes || n < 0 || temp_misaligned(temp) || (n > 0 && temp && (!in || !out))) return hipErrorInvalidValue;
  hipError_t rc = hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  bool ok = dispatch_dtype(dtype, [&](auto t) {
    using T = decltype(t);
    dispatch_op(op, [&](auto o) {
      using Op = decltype(o);
      rc = scan_typed<T, Op>(temp, temp_bytes, exclusive, in, out, n, init, s);
    });
  });
  (void)ok;
  return (int)rc;
}

// ---------------------------------------------------------------------------------------
// The same scan for callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): ticket and tile descriptors live in a fixed array in the
// library's device image instead of caller-provided temporary storage.
// ---------------------------------------------------------------------------------------
namespace tcd {
constexpr int64_t kStaticScanMaxTiles = 16384;  // tiles of 128 KiB: 2 GiB of input
constexpr size_t kStaticScanScratchBytes = 256 + (size_t)kStaticScanMaxTiles * 16;  // ticket + 16 B per tile
static __device__ __align__(256) unsigned char scratch[kStaticScanScratchBytes];

// `scratch` names the host-side stand-in of the symbol; the array's device address differs per
// GPU and is looked up once per device, with that device current.
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices];

static hipError_t static_scratch(void** out, hipStream_t stream) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    // the look-up is not something to do while the caller records a graph
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess) {
      (void)hipGetLastError();
      return hipErrorStreamCaptureUnsupported;
    }
    if (cs != hipStreamCaptureStatusNone) return hipErrorStreamCaptureUnsupported;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}
}  // namespace tcd

extern "C" int thrust_cdna4_scan_static(int dtype, int op, int exclusive, const void* in, void* out,
                                        int64_t n, const void* init, void* stream) {
  using namespace tcd;
  if (n < 0) return hipErrorInvalidValue;
  // The size limit is checked first and has its own code, whatever the pointers are.
  // (tiles the array has descriptors for: 16384, or 10922 for the three-word descriptors of a
  // minimum scan over 8-byte floating-point values)
  int64_t ntiles = -1, max_tiles = 0;
  dispatch_dtype(dtype, [&](auto t) {
    using T = decltype(t);
    dispatch_op(op, [&](auto o) {
      ntiles = ceil_div(n, ScanConfig<T>::TILE);
      max_tiles = (int64_t)((kStaticScanScratchBytes - 256) / TileDesc<typename scan_payload<T, decltype(o)>::type>::kBytesPerTile);
      if (max_tiles > kStaticScanMaxTiles) max_tiles = kStaticScanMaxTiles;
    });
  });
  if (ntiles < 0) return hipErrorInvalidValue;  // unknown element type or operator
  if (ntiles > max_tiles) return hipErrorOutOfMemory;
  if (n > 0 && (!in || !out)) return hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  void* ptr = nullptr;
  hipError_t rc = static_scratch(&ptr, s);
  if (rc != hipSuccess) return (int)rc;
  rc = hipErrorInvalidValue;
  dispatch_dtype(dtype, [&](auto t) {
    using T = decltype(t);
    dispatch_op(op, [&](auto o) {
      using Op = decltype(o);
      // scan_typed checks the size it needs against the bytes it is given and clears the
      // descriptors it will use with a fill kernel before the scan kernel reads them
      size_t bytes = kStaticScanScratchBytes;
      rc = scan_typed<T, Op>(ptr, &bytes, exclusive, in, out, n, init, s);
    });
  });
  return (int)rc;
}
