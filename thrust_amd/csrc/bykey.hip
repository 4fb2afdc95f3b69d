// Segmented single-pass kernels for gfx950: scan_by_key and reduce_by_key.
//
// Both run the same decoupled look-back engine as the plain scan, over pairs
// (number of segment heads, value): combine(a, b) = (a.c + b.c, b.c ? b.v : a.v (+) b.v).
// A head is an element whose key differs from its predecessor's (element 0 is a head).
//
//   scan_by_key     semantics thrust/system/detail/sequential/scan_by_key.h:46-142, replaces
//                   thrust/system/cuda/detail/scan_by_key.h:69-282 (cub::DispatchScanByKey)
//   reduce_by_key   semantics thrust/system/detail/sequential/reduce_by_key.h:43-95, replaces
//                   ReduceByKeyAgent / InitAgent, thrust/system/cuda/detail/reduce_by_key.h:204-1058
//
// This file is compiled once per key width (-DTCD_KEY_BYTES=1|2|4|8); keys are compared as
// bit patterns, or as IEEE numbers when `float_keys` is set (-0 == +0, NaN != NaN), which is
// what thrust::equal_to does.
#include "common.h"

#ifndef TCD_KEY_BYTES
#error "compile with -DTCD_KEY_BYTES=1|2|4|8"
#endif

#define TCD_CAT2(a, b) a##b
#define TCD_CAT(a, b) TCD_CAT2(a, b)

namespace tcd {
// One namespace per key width.  This file is compiled four times into one library, and the key
// type is a file-level alias, not a template argument: SegGeom<T>, SegTile<...> and the host
// helpers below differ between the four objects under one name.  Inside a namespace of their
// own no linker can fold a copy from one key width into another's.
inline namespace TCD_CAT(keys_of_bytes_, TCD_KEY_BYTES) {

template <int B> struct key_bits;
template <> struct key_bits<1> { using type = uint8_t; };
template <> struct key_bits<2> { using type = uint16_t; };
template <> struct key_bits<4> { using type = uint32_t; };
template <> struct key_bits<8> { using type = uint64_t; };
using KU = key_bits<TCD_KEY_BYTES>::type;

template <class T, bool RESTARTS = false>
struct SegPair {
  uint32_t c;  // heads seen
  T v;         // value of the open segment
};
// minimum(a, b) = a < b ? a : b over floating-point values with NaNs: the serial fold RESTARTS at
// every NaN (acc < NaN is false, so the NaN replaces the accumulator; NaN < x is false too, so the
// next element replaces the NaN).  The raw operator does that by itself wherever values are folded
// in input order; where PIECES are combined, a piece must also say whether it holds a NaN after its
// last head — nothing to its left survives that NaN, just as nothing survives a head.  And the
// empty piece needs a state of its own, because the operator's identity is none for a NaN
// (minimum(NaN, +inf) is +inf) and accumulators are shown as they are (the value of a run that
// ends with a NaN; exclusive scans).  Only the floating-point minimum instantiations carry this.
template <class T>
struct SegPair<T, true> {
  uint32_t c;  // heads seen
  uint32_t r;  // after the last head (or in all of a piece without one) — 0: no NaN, 1: a NaN; 2: the piece is empty
  T v;         // value of the open segment
};
template <class T, class Op>
struct seg_restarts {
  static constexpr bool value = std::is_floating_point<T>::value && std::is_same<Op, OpMinimum>::value;
};

template <class T, class Op>
__device__ inline SegPair<T> seg_combine(const SegPair<T>& a, const SegPair<T>& b) {
  SegPair<T> r;
  r.c = a.c + b.c;
  r.v = b.c ? b.v : Op::template apply<T>(a.v, b.v);
  return r;
}
template <class T, class Op>
__device__ inline SegPair<T, true> seg_combine(const SegPair<T, true>& a, const SegPair<T, true>& b) {
  if (b.r == 2u) return a;
  if (a.r == 2u) return b;
  SegPair<T, true> r;
  r.c = a.c + b.c;
  r.r = b.c ? b.r : (a.r | b.r);
  r.v = (b.c || b.r) ? b.v : Op::template apply<T>(a.v, b.v);
  return r;
}
// one more element at the end of a piece
template <class T, class Op>
__device__ inline void seg_append(SegPair<T>& a, bool is_head, T x) {
  a.c += is_head ? 1u : 0u;
  a.v = is_head ? x : Op::template apply<T>(a.v, x);
}
template <class T, class Op>
__device__ inline void seg_append(SegPair<T, true>& a, bool is_head, T x) {
  const bool fresh = is_head || a.r == 2u;
  a.c += is_head ? 1u : 0u;
  a.v = fresh ? x : Op::template apply<T>(a.v, x);
  a.r = (fresh ? 0u : a.r) | (__builtin_isnan(x) ? 1u : 0u);
}
template <class P, class T>
__device__ inline P seg_empty(T id) {
  P p;
  p.c = 0u;
  p.v = id;
  if constexpr (!std::is_same<P, SegPair<T>>::value) p.r = 2u;
  return p;
}

template <class KU>
__device__ inline bool keys_differ(KU a, KU b, int float_keys) {
  if constexpr (sizeof(KU) >= 4) {
    if (float_keys) {
      constexpr int W = 8 * sizeof(KU);
      const KU abs_a = KU(a << 1), abs_b = KU(b << 1);           // sign shifted out
      const KU exp_all = KU(~KU(0)) << (W == 32 ? 24 : 53);       // exponent all ones, <<1
      const bool nan_a = abs_a > exp_all, nan_b = abs_b > exp_all;
      const bool both_zero = (abs_a | abs_b) == 0;
      return nan_a || nan_b || !(a == b || both_zero);
    }
  }
  return a != b;
}

// Both kernels are compiled for 4 wavefronts per SIMD (at most 128 VGPRs): two 512-thread
// workgroups per CU.  Left alone, the register allocator may trade that occupancy away.
#define TCD_SEG_ATTR __attribute__((amdgpu_waves_per_eu(4)))
// Tile geometry: blocked tiles.  A thread owns VEC consecutive elements (128 bytes of the wider
// of key and value, at most 32 elements), a wavefront 64 * VEC consecutive ones.  Global memory is
// read and written in wave-wide contiguous 1 KiB accesses and transposed to the blocked order
// through a wave-private LDS buffer, so one sequential walk per thread and ONE wavefront scan per
// tile do the work.  (A striped layout, 16-byte groups of each of 8 chunks per thread with a scan
// per group, needed three times the vector instructions; at 2^28 int32 pairs it was 2 % faster
// when every element is a run of its own and 3-5 % slower at mean run lengths 8 and 512.)
template <class T>
struct SegGeom {
  static constexpr int BLOCK = 512;
  static constexpr int WIDE = (int)(sizeof(KU) > sizeof(T) ? sizeof(KU) : sizeof(T));
  static constexpr int VEC = WIDE == 8 ? 16 : 32;
  static constexpr int NWAVES = BLOCK / kWave;
  static constexpr int64_t TILE = (int64_t)BLOCK * VEC;
  static constexpr int XPOSE_SLOTS = 512;  // 16-byte slots of a wavefront's transpose buffer (8 KiB)
};

// Orders a wavefront's LDS accesses around an exchange through its private buffer (the LDS
// executes one wavefront's instructions in order; this keeps the compiler from reordering them).
__device__ inline void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// 16-byte slot s of a wavefront's buffer lives at slot xpose_slot(s): both the striped order
// (slot q * 64 + lane) and the blocked order (slot lane * NQ + i) then spread over all banks.
__device__ inline int xpose_slot(int s) { return s ^ ((s >> 3) & 7); }

// The wavefront's 64 * VEC consecutive elements at src (16-byte aligned): lane l receives
// elements [l * VEC, (l + 1) * VEC).  Every global access is one contiguous 1 KiB per wavefront.
template <int VEC, class E>
__device__ inline void wave_load_blocked(const E* src, E (&dst)[VEC], tcd_v4u* buf, int lane) {
  constexpr int NQ = VEC * (int)sizeof(E) / 16;
  static_assert(NQ >= 1 && NQ * 16 == VEC * (int)sizeof(E), "a thread's elements are whole 16-byte slots");
  tcd_v4u t[NQ];
#pragma unroll
  for (int q = 0; q < NQ; q++) t[q] = load16<tcd_v4u>(reinterpret_cast<const char*>(src) + (q * kWave + lane) * 16);
#pragma unroll
  for (int q = 0; q < NQ; q++) buf[xpose_slot(q * kWave + lane)] = t[q];
  wave_lds_sync();
#pragma unroll
  for (int i = 0; i < NQ; i++) {
    const tcd_v4u r = buf[xpose_slot(lane * NQ + i)];
    __builtin_memcpy(reinterpret_cast<char*>(dst) + 16 * i, &r, 16);
  }
  wave_lds_sync();
}
// The inverse: lane l's VEC consecutive elements go to dst[l * VEC ...], written as contiguous
// 1 KiB accesses.
template <int VEC, class E>
__device__ inline void wave_store_blocked(E* dst, const E (&src)[VEC], tcd_v4u* buf, int lane) {
  constexpr int NQ = VEC * (int)sizeof(E) / 16;
  static_assert(NQ >= 1 && NQ * 16 == VEC * (int)sizeof(E), "a thread's elements are whole 16-byte slots");
#pragma unroll
  for (int i = 0; i < NQ; i++) {
    tcd_v4u r;
    __builtin_memcpy(&r, reinterpret_cast<const char*>(src) + 16 * i, 16);
    buf[xpose_slot(lane * NQ + i)] = r;
  }
  wave_lds_sync();
#pragma unroll
  for (int q = 0; q < NQ; q++) store16(reinterpret_cast<char*>(dst) + (q * kWave + lane) * 16, buf[xpose_slot(q * kWave + lane)]);
  wave_lds_sync();
}
// The same for a wavefront whose elements end before its 64 * VEC-th: only `avail` elements exist
// at src (possibly none, possibly all).  16-byte pieces that exist entirely move as above, the one
// piece the end falls into is read or written element by element, the rest is zero / untouched.
template <int VEC, class E>
__device__ inline void wave_load_blocked_partial(const E* src, E (&dst)[VEC], tcd_v4u* buf, int lane, int64_t avail) {
  constexpr int NQ = VEC * (int)sizeof(E) / 16;
  constexpr int EPP = 16 / (int)sizeof(E);
  tcd_v4u t[NQ];
#pragma unroll
  for (int q = 0; q < NQ; q++) {
    const int64_t e0 = (int64_t)(q * kWave + lane) * EPP;
    t[q] = tcd_v4u{0u, 0u, 0u, 0u};
    if (e0 + EPP <= avail) {
      t[q] = load16<tcd_v4u>(reinterpret_cast<const char*>(src) + (q * kWave + lane) * 16);
    } else if (e0 < avail) {
      E part[EPP] = {};
      for (int e = 0; e < EPP; e++)
        if (e0 + e < avail) part[e] = src[e0 + e];
      __builtin_memcpy(&t[q], part, 16);
    }
  }
#pragma unroll
  for (int q = 0; q < NQ; q++) buf[xpose_slot(q * kWave + lane)] = t[q];
  wave_lds_sync();
#pragma unroll
  for (int i = 0; i < NQ; i++) {
    const tcd_v4u r = buf[xpose_slot(lane * NQ + i)];
    __builtin_memcpy(reinterpret_cast<char*>(dst) + 16 * i, &r, 16);
  }
  wave_lds_sync();
}
template <int VEC, class E>
__device__ inline void wave_store_blocked_partial(E* dst, const E (&src)[VEC], tcd_v4u* buf, int lane, int64_t avail) {
  constexpr int NQ = VEC * (int)sizeof(E) / 16;
  constexpr int EPP = 16 / (int)sizeof(E);
#pragma unroll
  for (int i = 0; i < NQ; i++) {
    tcd_v4u r;
    __builtin_memcpy(&r, reinterpret_cast<const char*>(src) + 16 * i, 16);
    buf[xpose_slot(lane * NQ + i)] = r;
  }
  wave_lds_sync();
#pragma unroll
  for (int q = 0; q < NQ; q++) {
    const int64_t e0 = (int64_t)(q * kWave + lane) * EPP;
    const tcd_v4u piece = buf[xpose_slot(q * kWave + lane)];
    if (e0 + EPP <= avail) {
      store16(reinterpret_cast<char*>(dst) + (q * kWave + lane) * 16, piece);
    } else if (e0 < avail) {
      E part[EPP];
      __builtin_memcpy(part, &piece, 16);
      for (int e = 0; e < EPP; e++)
        if (e0 + e < avail) dst[e0 + e] = part[e];
    }
  }
  wave_lds_sync();
}

// Loads a tile, finds the segment heads, reduces it and resolves the prefix of all earlier
// tiles by look-back.  On return key/val hold the thread's VEC consecutive elements, bit j of
// `heads` says whether element j starts a segment, and `off` is the pair (heads seen, value of the
// open segment) of everything before the thread's first element.  The kernels then walk their
// elements once more from `off`; nothing per element is kept in between.
template <class T, class Op, class G>
struct SegTile {
  static constexpr bool kRestarts = seg_restarts<T, Op>::value;
  using Pair = SegPair<T, kRestarts>;
  static constexpr int VEC = G::VEC, NWAVES = G::NWAVES, BLOCK = G::BLOCK;
  static_assert(NWAVES <= kWave, "one wavefront scans the wavefronts' totals");

  struct Smem {
    Pair tot[NWAVES];  // inclusive total of a wavefront, then its prefix over the whole input
    uint32_t tile;
  };

  KU key[VEC];
  T val[VEC];
  uint32_t heads;
  Pair excl_w;  // everything before the thread's elements within its wavefront
  Pair off;
  int64_t base;
  int64_t tile;
  bool full;  // every element of the tile exists, the tile is not the last one, pointers are aligned to their elements

  __device__ int64_t first_index() const { return base + (int64_t)threadIdx.x * VEC; }

  __device__ static Pair comb(const Pair& a, const Pair& b) { return seg_combine<T, Op>(a, b); }

  // xbuf: the wavefront's transpose buffer.  TICKET: tiles are handed out by an atomic counter
  // (every tile waited for has started; used when an output overlaps an input); otherwise a tile
  // is the workgroup of the same index and a descriptor that stays missing after `patience` polls
  // is recomputed from the input.
  // maximum(a, b) = a < b ? b : a over floating-point values with NaNs is not associative: the
  // serial fold keeps a NaN that STARTS it (NaN < x is false) and skips a NaN met later
  // (acc < NaN is false too).  A NaN that cannot start a fold is therefore replaced by the
  // identity as the elements are classified — every NaN but those of segment heads; and those
  // too when `folds_start_from_init` (exclusive_scan_by_key, whose folds start from `init`).  What
  // is left is associative, and a NaN only ever appears as the operator's LEFT operand, where it
  // is kept.  Nothing of this is compiled for other types and operators.
  static constexpr bool kNanAware = std::is_floating_point<T>::value && std::is_same<Op, OpMaximum>::value;

  template <bool TICKET, class Meanwhile>
  __device__ void run(Smem& sm, const KU* keys, const T* vals, int64_t n, int float_keys, int vec_ok,
                      uint64_t* desc, uint32_t* ticket, tcd_v4u* xbuf, int patience, int publish_delay,
                      bool folds_start_from_init, Meanwhile meanwhile) {
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const T id = Op::template identity<T>();
    const Pair idp = seg_empty<Pair>(id);

    tile = blockIdx.x;
    if constexpr (TICKET) {
      if (tid == 0) sm.tile = atomicAdd(ticket, 1u);
      __syncthreads();
      tile = sm.tile;
    }
    base = tile * G::TILE;
    full = vec_ok && (base + G::TILE < n);

    if (full) {
      const int64_t w0 = base + (int64_t)wave * (kWave * VEC);
      wave_load_blocked<VEC>(keys + w0, key, xbuf, lane);
      wave_load_blocked<VEC>(vals + w0, val, xbuf, lane);
    } else if (vec_ok) {
      // the last tile: the same contiguous accesses up to the end of the input; elements that
      // do not exist read as key 0 and the operator's identity
      const int64_t w0 = base + (int64_t)wave * (kWave * VEC);
      wave_load_blocked_partial<VEC>(keys + w0, key, xbuf, lane, n - w0);
      wave_load_blocked_partial<VEC>(vals + w0, val, xbuf, lane, n - w0);
      const int64_t i0 = first_index();
#pragma unroll
      for (int j = 0; j < VEC; j++)
        if (i0 + j >= n) val[j] = id;
    } else {
      const int64_t i0 = first_index();
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        const int64_t idx = i0 + j;
        key[j] = idx < n ? keys[idx] : KU(0);
        val[j] = idx < n ? vals[idx] : id;
      }
    }
    // the key before a thread's elements is the last key of the lane below (its elements precede
    // these in memory); only lane 0 of each wave fetches it from memory
    using KW = typename std::conditional<(sizeof(KU) < 4), uint32_t, KU>::type;
    // (the index is formed here, after the loads: held across them it costs the by-key kernels
    // their register budget)
    const int64_t i0 = first_index();
    KU first = KU(0);
    if (lane == 0 && i0 > 0 && i0 < n) first = keys[i0 - 1];
    const KU prev = (KU)wave_shift_up1((KW)key[VEC - 1], (KW)first);

    {
      uint32_t h = 0;
      Pair agg = idp;
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        const KU p = j == 0 ? prev : key[j - 1];
        const bool is_head = (full || i0 + j < n) && (i0 + j == 0 || keys_differ(p, key[j], float_keys));
        if constexpr (kNanAware) {
          if ((folds_start_from_init || !is_head) && __builtin_isnan(val[j])) val[j] = id;
        }
        h |= (is_head ? 1u : 0u) << j;
        if constexpr (kRestarts) seg_append<T, Op>(agg, is_head, val[j]);
        else agg.v = is_head ? val[j] : Op::template apply<T>(agg.v, val[j]);
      }
      heads = h;
      if constexpr (!kRestarts) agg.c = __builtin_popcount(h);
      const Pair w = wave_inclusive_scan(agg, idp, comb);
      excl_w = wave_shift_up1(w, idp);
      if (lane == kWave - 1) sm.tot[wave] = w;
    }
    __syncthreads();

    // wave 0: scan of the wavefronts' totals in tile order, look-back, then each wavefront's
    // prefix over the whole input goes back into the table
    Pair tile_agg = idp, before = idp;
    if (wave == 0) {
      const Pair mine = lane < NWAVES ? sm.tot[lane] : idp;
      const Pair incl = wave_inclusive_scan(mine, idp, comb);
      tile_agg = readlane(incl, kWave - 1);
      before = wave_shift_up1(incl, idp);
      if (tile == 0)
        for (int i = 0; i < publish_delay; i++) __builtin_amdgcn_s_sleep(127);  // test knob, 0 in normal use
      if (lane == 0) TileDesc<Pair>::store(desc, tile, tile == 0 ? kInclusive : kPartial, tile_agg);
    }
    // work that needs nothing from earlier tiles runs while their aggregates arrive
    meanwhile();
    if (wave == 0) {
      Pair prefix = idp;
      if (tile != 0) {
        if constexpr (TICKET) {
          prefix = wave_lookback<Pair>(desc, tile, idp, comb);
        } else {
          // the aggregate of an earlier tile (always a whole one), straight from the input: each
          // lane folds a contiguous piece, the pieces combine in lane order
          const auto aggregate_of = [&](int64_t t) -> Pair {
            constexpr int PIECE = (int)(G::TILE / kWave);
            const int64_t start = t * G::TILE + (int64_t)lane * PIECE;
            KU before = start > 0 ? keys[start - 1] : KU(0);
            Pair a = idp;
            for (int k = 0; k < PIECE; k++) {
              const KU kk = keys[start + k];
              T vv = vals[start + k];
              const bool is_head = start + k == 0 || keys_differ(before, kk, float_keys);
              if constexpr (kNanAware) {
                if ((folds_start_from_init || !is_head) && __builtin_isnan(vv)) vv = Op::template identity<T>();
              }
              seg_append<T, Op>(a, is_head, vv);
              before = kk;
            }
            return readlane(wave_inclusive_scan(a, idp, comb), kWave - 1);
          };
          prefix = wave_lookback_or_compute<Pair>(desc, tile, idp, comb, patience, aggregate_of);
        }
        if (lane == 0) TileDesc<Pair>::store(desc, tile, kInclusive, comb(prefix, tile_agg));
      }
      if (lane < NWAVES) sm.tot[lane] = comb(prefix, before);
    }
    __syncthreads();
    off = comb(sm.tot[wave], excl_w);
  }
};

// ---------------------------------------------------------------------------------------
// scan_by_key
// ---------------------------------------------------------------------------------------
template <class T, class Op, bool TICKET>
__global__ __launch_bounds__(SegGeom<T>::BLOCK) TCD_SEG_ATTR void scan_by_key_kernel(
    const KU* keys, const T* vals, T* out, int64_t n, T init, int exclusive, int float_keys, int vec_ok,
    uint64_t* desc, uint32_t* ticket, int patience, int publish_delay) {
  using G = SegGeom<T>;
  using ST = SegTile<T, Op, G>;
  __shared__ typename ST::Smem sm;
  __shared__ tcd_v4u s_x[G::NWAVES][G::XPOSE_SLOTS];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  tcd_v4u* xbuf = s_x[wave];
  ST t;
  constexpr int VEC = ST::VEC;
  // Whole tiles: each wavefront scans its elements from the wavefront's own start and parks the
  // result in its buffer (in the order of the later contiguous stores) BEFORE the look-back.
  // Afterwards only the elements of the run that came into the wavefront open (those before its
  // first head, `first_head` of them) still take the value of that run so far; the four operators
  // are commutative, so it is applied on top of the parked result.
  constexpr int NQ = VEC * (int)sizeof(T) / 16;
  constexpr int EPP = 16 / (int)sizeof(T);  // elements per 16-byte slot
  bool parked = false;
  uint32_t first_head = 0;
  t.template run<TICKET>(sm, keys, vals, n, float_keys, vec_ok, desc, ticket, xbuf, patience, publish_delay, exclusive != 0, [&] {
    // (a restarting fold is not commutative: its tiles all take the walk from the tile's prefix below)
    if (!t.full || ST::kRestarts) return;
    parked = true;
    T r[VEC];
    T open = t.excl_w.v;
    // Floating-point maximum keeps the FIRST of +0 and -0: an exclusive result before the
    // wavefront's first head is init (+) run so far (+) wavefront's fold, in that order, so `init`
    // is left out of what is parked there and goes in front during the copy-out.
    bool none_below = false;  // no head in the lanes below
    if constexpr (ST::kNanAware) none_below = exclusive && !(__ballot(t.heads != 0u) & ((1ull << lane) - 1ull));
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      const bool is_head = (t.heads >> j) & 1u;
      const T x = t.val[j];
      const bool before_first_head = ST::kNanAware && none_below && !(t.heads & ((2u << j) - 1u));
      if (exclusive) r[j] = is_head ? init : before_first_head ? open : Op::template apply<T>(init, open);
      open = is_head ? x : Op::template apply<T>(open, x);
      if (!exclusive) r[j] = open;
    }
    const uint64_t has = __ballot(t.heads != 0u);
    first_head = kWave * VEC;
    if (has) {
      const int owner = __builtin_ctzll(has);
      first_head = (uint32_t)(owner * VEC + __builtin_ctz((uint32_t)__builtin_amdgcn_readlane((int)t.heads, owner)));
    }
#pragma unroll
    for (int i = 0; i < NQ; i++) {
      tcd_v4u piece;
      __builtin_memcpy(&piece, reinterpret_cast<const char*>(r) + 16 * i, 16);
      xbuf[xpose_slot(lane * NQ + i)] = piece;
    }
  });
  if (parked) {
    const T carried = sm.tot[wave].v;  // the open run's value over everything before the wavefront
    char* dst = reinterpret_cast<char*>(out + t.base + (int64_t)wave * (kWave * VEC));
#pragma unroll
    for (int q = 0; q < NQ; q++) {
      tcd_v4u piece = xbuf[xpose_slot(q * kWave + lane)];
      if ((uint32_t)(q * kWave * EPP) < first_head) {  // wave-uniform
        T x[EPP];
        __builtin_memcpy(x, &piece, 16);
#pragma unroll
        for (int e = 0; e < EPP; e++)
          if ((uint32_t)((q * kWave + lane) * EPP + e) < first_head) {
            // the run's value so far goes in front of what the wavefront folded; the exclusive
            // form has `init` in front of both: already inside x[e] where the operands commute,
            // applied here in fold order where they do not (floating-point maximum: a NaN, or
            // +0 against -0)
            if constexpr (ST::kNanAware) {
              x[e] = Op::template apply<T>(carried, x[e]);
              if (exclusive) x[e] = Op::template apply<T>(init, x[e]);
            } else {
              x[e] = exclusive ? Op::template apply<T>(x[e], carried) : Op::template apply<T>(carried, x[e]);
            }
          }
        __builtin_memcpy(&piece, x, 16);
      }
      store16(dst + (q * kWave + lane) * 16, piece);
    }
    return;
  }
  // the last tile, and every tile of a call whose pointers are not aligned to their elements
  T r[VEC];
  T open = t.off.v;  // value of the open segment just before the element
  if constexpr (ST::kRestarts) {
    // the raw fold restarts at NaNs by itself; `init` of an exclusive scan is in front of the
    // fold only until the segment's first NaN
    bool restarted = t.off.r == 1u;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      const bool is_head = (t.heads >> j) & 1u;
      const T x = t.val[j];
      if (exclusive) r[j] = is_head ? init : restarted ? open : Op::template apply<T>(init, open);
      open = is_head ? x : Op::template apply<T>(open, x);
      restarted = (!is_head && restarted) || __builtin_isnan(x);
      if (!exclusive) r[j] = open;
    }
  } else {
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      const bool is_head = (t.heads >> j) & 1u;
      const T x = t.val[j];
      if (exclusive) r[j] = is_head ? init : Op::template apply<T>(init, open);
      open = is_head ? x : Op::template apply<T>(open, x);
      if (!exclusive) r[j] = open;
    }
  }
  if (vec_ok) {
    const int64_t w0 = t.base + (int64_t)wave * (kWave * VEC);
    wave_store_blocked_partial<VEC>(out + w0, r, xbuf, lane, n - w0);
  } else {
    const int64_t i0 = t.first_index();
#pragma unroll
    for (int j = 0; j < VEC; j++)
      if (i0 + j < n) out[i0 + j] = r[j];
  }
}

// ---------------------------------------------------------------------------------------
// reduce_by_key
// ---------------------------------------------------------------------------------------
template <class T, class Op, bool TICKET>
__global__ __launch_bounds__(SegGeom<T>::BLOCK) TCD_SEG_ATTR void reduce_by_key_kernel(
    const KU* keys, const T* vals, KU* keys_out, T* vals_out, int64_t* num_runs, int64_t n,
    int float_keys, int vec_ok, uint64_t* desc, uint32_t* ticket, int patience, int publish_delay) {
  using G = SegGeom<T>;
  using ST = SegTile<T, Op, G>;
  constexpr int VEC = ST::VEC, NWAVES = ST::NWAVES;
  __shared__ typename ST::Smem sm;
  const int lane = threadIdx.x & (kWave - 1);
  // The heads of a wavefront's 64 * VEC consecutive elements go to consecutive output slots.
  // They are compacted in the wavefront's buffer — keys first, then, through the same 8 KiB,
  // the values of the runs they close — and written with contiguous stores.
  static_assert(kWave * VEC * sizeof(KU) <= G::XPOSE_SLOTS * 16 && kWave * VEC * sizeof(T) <= G::XPOSE_SLOTS * 16,
                "a wavefront's heads fit its buffer");
  __shared__ tcd_v4u s_x[NWAVES][G::XPOSE_SLOTS];
  tcd_v4u* xbuf = s_x[threadIdx.x / kWave];
  ST t;
  // Slot i lives at sw(i): when most elements are heads a thread's slots start VEC apart, which
  // is one LDS bank for all lanes; the swizzle (within aligned groups of VEC slots) spreads them
  // and the copy-out reads over all banks.
  constexpr uint32_t kLogVec = VEC == 32 ? 5 : 4;
  static_assert((1u << kLogVec) == (uint32_t)VEC, "VEC is 16 or 32");
  const auto sw = [](uint32_t i) { return i ^ ((i >> kLogVec) & (uint32_t)(VEC - 1)); };
  // A wavefront with few enough heads compacts them BEFORE the look-back, while the aggregates
  // of earlier tiles are still on their way: keys into the lower half of its buffer, the values
  // of the runs they close into the upper half.  Only the output position and the start of the
  // run open at the wavefront's first element depend on earlier tiles; both are applied during
  // the copy-out.  (Not in the last tile, which also closes the last run.)
  constexpr uint32_t kHalfBytes = G::XPOSE_SLOTS * 16 / 2;
  constexpr uint32_t kEarlyMax = kHalfBytes / (sizeof(KU) > sizeof(T) ? sizeof(KU) : sizeof(T)) - VEC;
  KU* const early_k = reinterpret_cast<KU*>(xbuf);
  T* const early_v = reinterpret_cast<T*>(reinterpret_cast<char*>(xbuf) + kHalfBytes);
  bool early = false;
  uint32_t count = 0;
  t.template run<TICKET>(sm, keys, vals, n, float_keys, vec_ok, desc, ticket, xbuf, patience, publish_delay, false, [&] {
    count = (uint32_t)__builtin_amdgcn_readlane((int)(t.excl_w.c + __builtin_popcount(t.heads)), kWave - 1);
    early = t.full && count <= kEarlyMax && !ST::kRestarts;  // (the early form counts on a commutative operator)
    if (!early) {
      if (t.full) {  // the keys alone always fit
        uint32_t slot = t.excl_w.c;
#pragma unroll
        for (int j = 0; j < VEC; j++)
          if ((t.heads >> j) & 1u) early_k[sw(slot++)] = t.key[j];
      }
      return;
    }
    uint32_t slot = t.excl_w.c;
    T open = t.excl_w.v;  // the open run's value over the wavefront's earlier elements
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      if ((t.heads >> j) & 1u) {
        early_k[sw(slot)] = t.key[j];
        early_v[sw(slot)] = open;
        slot++;
        open = t.val[j];
      } else {
        open = Op::template apply<T>(open, t.val[j]);
      }
    }
  });
  if (early) {
    const typename ST::Pair before_wave = sm.tot[threadIdx.x / kWave];
    const uint32_t first = before_wave.c;
    for (uint32_t i = lane; i < count; i += kWave) {
      keys_out[first + i] = early_k[sw(i)];
      T v = early_v[sw(i)];
      if (i == 0) v = Op::template apply<T>(before_wave.v, v);  // the run came into the wavefront open
      if (first + i) vals_out[first + i - 1] = v;
    }
    return;
  }
  typename ST::Pair run = t.off;  // (runs started so far, value of the open run) before the current element
  const uint32_t first = (uint32_t)__builtin_amdgcn_readfirstlane((int)run.c);  // runs before this wavefront
  const uint32_t heads = t.heads;
  const uint32_t mine = run.c - first;  // slot of this thread's first head
  const int64_t i0 = t.first_index();
  // Too many heads for both halves (or the last tile): the values go through the buffer after
  // the keys.  A whole tile's keys were compacted before the look-back.
  KU* sk = reinterpret_cast<KU*>(xbuf);
  if (!t.full) {
    uint32_t slot = mine;
#pragma unroll
    for (int j = 0; j < VEC; j++)
      if ((heads >> j) & 1u) sk[sw(slot++)] = t.key[j];
  }
  wave_lds_sync();
  for (uint32_t i = lane; i < count; i += kWave) keys_out[first + i] = sk[sw(i)];
  wave_lds_sync();
  T* sv = reinterpret_cast<T*>(xbuf);
  {
    uint32_t slot = mine;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      const bool exists = t.full || i0 + j < n;
      if ((heads >> j) & 1u) {
        // a head closes the run before it and opens run number run.c
        sv[sw(slot++)] = run.v;
        run.c += 1;
        run.v = t.val[j];
      } else if (exists) {
        run.v = Op::template apply<T>(run.v, t.val[j]);
      }
      if (!t.full && i0 + j == n - 1) {  // the last element closes the last run
        vals_out[run.c - 1] = run.v;
        *num_runs = (int64_t)run.c;
      }
    }
  }
  wave_lds_sync();
  for (uint32_t i = lane; i < count; i += kWave)
    if (first + i) vals_out[first + i - 1] = sv[sw(i)];  // value of the run that ended at this head
}

template <class T, class Op, class G>
static size_t bykey_temp_bytes(int64_t n) {
  const int64_t ntiles = ceil_div(n, G::TILE);
  return 256 + align_up((size_t)ntiles * TileDesc<SegPair<T, seg_restarts<T, Op>::value>>::kBytesPerTile, 256);
}

}  // namespace keys_of_bytes_<width>
}  // namespace tcd

// Internal entry points, one pair per key width; the public C ABI in bykey_dispatch.hip
// selects by key dtype.
extern "C" int TCD_CAT(tcd_scan_by_key_k, TCD_KEY_BYTES)(void* temp, size_t* temp_bytes, int float_keys,
                                                         int value_dtype, int op, int exclusive,
                                                         const void* keys, const void* values, void* out,
                                                         int64_t n, const void* init, void* stream) {
  using namespace tcd;
  hipError_t rc = hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dispatch_dtype(value_dtype, [&](auto tv) {
    using T = decltype(tv);
    dispatch_op(op, [&](auto o) {
      using Op = decltype(o);
      const int64_t ntiles = ceil_div(n, SegGeom<T>::TILE);
      // one tile consults no descriptor and reads all its input before it writes: no clearing
      // launch, no tickets
      const bool single = ntiles <= 1;
      // An output over the KEYS: a tile reads the key before its first element from memory, where
      // the tile before it may already have written results.  The keys are then read from a copy
      // in the temporary storage (which is why the size query takes the same pointers as the call).
      const size_t desc_bytes = bykey_temp_bytes<T, Op, SegGeom<T>>(n);
      const bool keys_copied = !single && keys && out && ranges_overlap(out, (size_t)n * sizeof(T), keys, (size_t)n * sizeof(KU));
      const size_t need = desc_bytes + (keys_copied ? align_up((size_t)n * sizeof(KU), 256) : 0);
      if (!temp) { *temp_bytes = need; rc = hipSuccess; return; }
      if (*temp_bytes < need) return;
      if (n == 0) { rc = hipSuccess; return; }
      if (!single) {
        rc = zero_async(temp, desc_bytes, s);
        if (rc != hipSuccess) return;
      }
      if (keys_copied) {
        void* copy = static_cast<char*>(temp) + desc_bytes;
        rc = copy_async(copy, keys, (size_t)n * sizeof(KU), s);
        if (rc != hipSuccess) return;
        keys = copy;
      }
      T iv = T(0);
      if (init) __builtin_memcpy(&iv, init, sizeof(T));
      // 128-bit accesses need no more than the elements' own alignment (see load16)
      const int vec_ok = (reinterpret_cast<uintptr_t>(keys) & (sizeof(KU) - 1)) == 0 &&
                         ((reinterpret_cast<uintptr_t>(values) | reinterpret_cast<uintptr_t>(out)) & (sizeof(T) - 1)) == 0;
      // an output that overlaps the values: tiles by ticket
      const bool aliased = !single && ranges_overlap(out, (size_t)n * sizeof(T), values, (size_t)n * sizeof(T));
      if (aliased) {
        TCD_LAUNCH("scan_by_key_kernel", (scan_by_key_kernel<T, Op, true>), dim3((unsigned)ntiles), dim3(SegGeom<T>::BLOCK), s,
                           static_cast<const KU*>(keys), static_cast<const T*>(values), static_cast<T*>(out),
                           n, iv, exclusive, float_keys, vec_ok,
                           reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256),
                           reinterpret_cast<uint32_t*>(temp), 0, 0);
      } else {
        TCD_LAUNCH("scan_by_key_kernel", (scan_by_key_kernel<T, Op, false>), dim3((unsigned)ntiles), dim3(SegGeom<T>::BLOCK), s,
                           static_cast<const KU*>(keys), static_cast<const T*>(values), static_cast<T*>(out),
                           n, iv, exclusive, float_keys, vec_ok,
                           reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256),
                           reinterpret_cast<uint32_t*>(temp), lookback_patience(), lookback_test_publish_delay());
      }
      rc = hipGetLastError();
    });
  });
  return (int)rc;
}

extern "C" int TCD_CAT(tcd_reduce_by_key_k, TCD_KEY_BYTES)(void* temp, size_t* temp_bytes, int float_keys,
                                                           int value_dtype, int op, const void* keys_in,
                                                           const void* values_in, void* keys_out,
                                                           void* values_out, int64_t* num_runs_out,
                                                           int64_t n, void* stream) {
  using namespace tcd;
  hipError_t rc = hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dispatch_dtype(value_dtype, [&](auto tv) {
    using T = decltype(tv);
    dispatch_op(op, [&](auto o) {
      using Op = decltype(o);
      const int64_t ntiles = ceil_div(n, SegGeom<T>::TILE);
      const bool single = ntiles <= 1;  // as in scan_by_key
      // an output over the input keys: the keys are read from a copy, as in scan_by_key
      const size_t kb = (size_t)n * sizeof(KU), vb = (size_t)n * sizeof(T);
      const size_t desc_bytes = bykey_temp_bytes<T, Op, SegGeom<T>>(n);
      const bool keys_copied = !single && keys_in && ((keys_out && ranges_overlap(keys_out, kb, keys_in, kb)) ||
                                                       (values_out && ranges_overlap(values_out, vb, keys_in, kb)));
      const size_t need = desc_bytes + (keys_copied ? align_up(kb, 256) : 0);
      if (!temp) { *temp_bytes = need; rc = hipSuccess; return; }
      if (*temp_bytes < need) return;
      if (n == 0) {  // no runs: only the count is written
        rc = zero_async(num_runs_out, sizeof(int64_t), s);
        return;
      }
      if (!single) {
        rc = zero_async(temp, desc_bytes, s);
        if (rc != hipSuccess) return;
      }
      if (keys_copied) {
        void* copy = static_cast<char*>(temp) + desc_bytes;
        rc = copy_async(copy, keys_in, kb, s);
        if (rc != hipSuccess) return;
        keys_in = copy;
      }
      // 128-bit accesses need no more than the elements' own alignment (see load16)
      const int vec_ok = (reinterpret_cast<uintptr_t>(keys_in) & (sizeof(KU) - 1)) == 0 &&
                         (reinterpret_cast<uintptr_t>(values_in) & (sizeof(T) - 1)) == 0;
      // an output that overlaps the input values: tiles by ticket (a tile writes to the left of
      // its own elements only, where every tile has read its input before this one's look-back ends)
      const bool aliased = !single && (ranges_overlap(keys_out, kb, values_in, vb) || ranges_overlap(values_out, vb, values_in, vb));
      if (aliased) {
        TCD_LAUNCH("reduce_by_key_kernel", (reduce_by_key_kernel<T, Op, true>), dim3((unsigned)ntiles), dim3(SegGeom<T>::BLOCK), s,
                           static_cast<const KU*>(keys_in), static_cast<const T*>(values_in),
                           static_cast<KU*>(keys_out), static_cast<T*>(values_out), num_runs_out, n, float_keys,
                           vec_ok, reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256),
                           reinterpret_cast<uint32_t*>(temp), 0, 0);
      } else {
        TCD_LAUNCH("reduce_by_key_kernel", (reduce_by_key_kernel<T, Op, false>), dim3((unsigned)ntiles), dim3(SegGeom<T>::BLOCK), s,
                           static_cast<const KU*>(keys_in), static_cast<const T*>(values_in),
                           static_cast<KU*>(keys_out), static_cast<T*>(values_out), num_runs_out, n, float_keys,
                           vec_ok, reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256),
                           reinterpret_cast<uint32_t*>(temp), lookback_patience(), lookback_test_publish_delay());
      }
      rc = hipGetLastError();
    });
  });
  return (int)rc;
}
