// Device-side building blocks shared by the gfx950 kernels: wave64 DPP scans, tile
// descriptors for decoupled look-back, element-type dispatch.  CDNA4 only: a wavefront is
// 64 lanes, DPP row_bcast is available, L2 is per XCD so cross-workgroup communication goes
// through agent-scope atomics.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <type_traits>

#include "thrust_cdna4.h"

namespace tcd {

constexpr int kWave = 64;

// ---------------------------------------------------------------------------------------
// Bit casts and small helpers
// ---------------------------------------------------------------------------------------
template <class To, class From>
__host__ __device__ inline To bit_cast(const From& f) {
  static_assert(sizeof(To) == sizeof(From), "bit_cast size mismatch");
  To t;
  __builtin_memcpy(&t, &f, sizeof(To));
  return t;
}

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

__device__ inline int lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// ---------------------------------------------------------------------------------------
// Binary operators (thrust/functional.h: plus, multiplies, maximum, minimum).
// Integer arithmetic runs in the unsigned type of the same width so that overflow wraps.
// maximum(a,b) = a < b ? b : a; minimum(a,b) = a < b ? a : b, as the reference defines them.
// identity() is a left and right identity for every non-NaN value; for floating-point plus
// it is -0.0 (x + -0.0 == x bit for bit, which +0.0 does not give for x == -0.0).
// ---------------------------------------------------------------------------------------
template <class T>
struct unsigned_of {
  using type = typename std::make_unsigned<T>::type;
};
template <>
struct unsigned_of<float> {
  using type = uint32_t;
};
template <>
struct unsigned_of<double> {
  using type = uint64_t;
};

template <class T>
struct limits_of {
  __host__ __device__ static constexpr T lowest() {
    if constexpr (std::is_floating_point<T>::value)
      return -__builtin_huge_val();
    else if constexpr (std::is_signed<T>::value)
      return T(T(1) << (8 * sizeof(T) - 1));
    else
      return T(0);
  }
  __host__ __device__ static constexpr T highest() {
    if constexpr (std::is_floating_point<T>::value)
      return __builtin_huge_val();
    else if constexpr (std::is_signed<T>::value)
      return T(~(T(1) << (8 * sizeof(T) - 1)));
    else
      return T(~T(0));
  }
};

struct OpPlus {
  template <class T>
  __host__ __device__ static T apply(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
      using U = typename unsigned_of<T>::type;
      return T(U(U(a) + U(b)));
    } else {
      return a + b;
    }
  }
  template <class T>
  __host__ __device__ static T identity() {
    if constexpr (std::is_integral<T>::value) return T(0);
    else return T(-0.0);
  }
};
struct OpMultiplies {
  template <class T>
  __host__ __device__ static T apply(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
      using U = typename unsigned_of<T>::type;
      return T(U(U(a) * U(b)));
    } else {
      return a * b;
    }
  }
  template <class T>
  __host__ __device__ static T identity() { return T(1); }
};
struct OpMaximum {
  template <class T>
  __host__ __device__ static T apply(T a, T b) { return a < b ? b : a; }
  template <class T>
  __host__ __device__ static T identity() { return limits_of<T>::lowest(); }
};
struct OpMinimum {
  template <class T>
  __host__ __device__ static T apply(T a, T b) { return a < b ? a : b; }
  template <class T>
  __host__ __device__ static T identity() { return limits_of<T>::highest(); }
};

// ---------------------------------------------------------------------------------------
// DPP data movement for trivially copyable types whose size is a multiple of 4 bytes.
// Lanes whose DPP source is out of range or masked keep `old`.
// ---------------------------------------------------------------------------------------
constexpr int kDppRowShr0 = 0x110;
constexpr int kDppRowBcast15 = 0x142;
constexpr int kDppRowBcast31 = 0x143;

template <int CTRL, int ROW_MASK, class T>
__device__ inline T dpp_move(const T& old, const T& src) {
  static_assert(sizeof(T) % 4 == 0, "dpp_move needs whole dwords");
  constexpr int NW = sizeof(T) / 4;
  uint32_t o[NW], s[NW], r[NW];
  __builtin_memcpy(o, &old, sizeof(T));
  __builtin_memcpy(s, &src, sizeof(T));
#pragma unroll
  for (int i = 0; i < NW; i++)
    r[i] = (uint32_t)__builtin_amdgcn_update_dpp((int)o[i], (int)s[i], CTRL, ROW_MASK, 0xf, false);
  T out;
  __builtin_memcpy(&out, r, sizeof(T));
  return out;
}

template <class T>
__device__ inline T readlane(const T& v, int lane) {
  static_assert(sizeof(T) % 4 == 0, "readlane needs whole dwords");
  constexpr int NW = sizeof(T) / 4;
  uint32_t s[NW], r[NW];
  __builtin_memcpy(s, &v, sizeof(T));
#pragma unroll
  for (int i = 0; i < NW; i++) r[i] = (uint32_t)__builtin_amdgcn_readlane((int)s[i], lane);
  T out;
  __builtin_memcpy(&out, r, sizeof(T));
  return out;
}

// Inclusive scan across the 64 lanes of a wavefront: lane i gets x[0] (+) ... (+) x[i],
// where a (+) b = f(a, b).  Every lane of the wave must be active.  `id` must be an
// identity of f.  Four row_shr steps scan each row of 16 lanes, row_bcast15 carries rows
// 0→1 and 2→3, row_bcast31 carries the lower half into the upper half.
template <class T, class F>
__device__ inline T wave_inclusive_scan(T v, const T id, F f) {
  v = f(dpp_move<kDppRowShr0 | 1, 0xf>(id, v), v);
  v = f(dpp_move<kDppRowShr0 | 2, 0xf>(id, v), v);
  v = f(dpp_move<kDppRowShr0 | 4, 0xf>(id, v), v);
  v = f(dpp_move<kDppRowShr0 | 8, 0xf>(id, v), v);
  v = f(dpp_move<kDppRowBcast15, 0xa>(id, v), v);
  v = f(dpp_move<kDppRowBcast31, 0xc>(id, v), v);
  return v;
}

// Exclusive value of lane i from an inclusive scan: the inclusive value of lane i-1
// (fetched with ds_bpermute), or `id` in lane 0.
template <class T>
__device__ inline T wave_shift_up1(const T& incl, const T id) {
  static_assert(sizeof(T) % 4 == 0, "whole dwords");
  constexpr int NW = sizeof(T) / 4;
  uint32_t s[NW], r[NW];
  __builtin_memcpy(s, &incl, sizeof(T));
  const int lane = lane_id();
#pragma unroll
  for (int i = 0; i < NW; i++)
    r[i] = (uint32_t)__builtin_amdgcn_ds_bpermute((lane - 1) << 2, (int)s[i]);
  T out;
  __builtin_memcpy(&out, r, sizeof(T));
  return lane == 0 ? id : out;
}

// 16-byte streaming accesses.  Data that a kernel touches exactly once is loaded and stored
// with the non-temporal hint, which keeps it from displacing other lines in the L2 (scan and
// by-key kernels gain 3-4 %).  The sort's scattered 4- and 8-byte stores must NOT use it: they
// rely on the L2 to merge the pieces of a line written by different waves (measured 25 % slower).
typedef unsigned int tcd_v4u __attribute__((ext_vector_type(4)));
// The same 16 bytes at ANY address in global memory: gfx950 under the HSA ABI runs with unaligned
// global access enabled, and the compiler emits the one 128-bit instruction for this type as it
// does for the aligned one.  load16 / store16 use it, so a range that starts a few elements into
// an allocation (v.begin() + 1) takes the same vector paths as an aligned one; only LDS accesses
// go through the aligned tcd_v4u.
typedef tcd_v4u tcd_v4u_anywhere __attribute__((aligned(1)));
template <class V, class E>
__device__ inline V load16(const E* p) {
  static_assert(sizeof(V) == 16, "16-byte vector");
  tcd_v4u r;
  r = __builtin_nontemporal_load(reinterpret_cast<const tcd_v4u_anywhere*>(p));
  V v;
  __builtin_memcpy(&v, &r, 16);
  return v;
}
template <class V, class E>
__device__ inline void store16(E* p, const V& v) {
  static_assert(sizeof(V) == 16, "16-byte vector");
  tcd_v4u r;
  __builtin_memcpy(&r, &v, 16);
  __builtin_nontemporal_store(r, reinterpret_cast<tcd_v4u_anywhere*>(p));
}

// ---------------------------------------------------------------------------------------
// Tile descriptors for decoupled look-back.
//
// A payload of NW 32-bit words is stored as NW 64-bit atoms, each (status << 32 | word).
// Status and data travel in ONE naturally aligned 64-bit relaxed agent-scope atomic, so no
// fence is needed between "write the value" and "raise the flag", and a reader that sees the
// same status in all NW atoms has a consistent payload (each atom is written once per
// status).  Agent scope makes the accesses coherent across the 8 XCD-private L2s.
// ---------------------------------------------------------------------------------------
enum : uint32_t { kInvalid = 0, kPartial = 1, kInclusive = 2 };

__device__ inline uint64_t ld_agent(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void st_agent(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline uint32_t ld_agent(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void st_agent(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// P is a trivially copyable payload; it is padded to whole dwords.
template <class P>
struct TileDesc {
  static constexpr int NW = (sizeof(P) + 3) / 4;
  static constexpr size_t kBytesPerTile = NW * sizeof(uint64_t);

  __device__ static void store(uint64_t* base, int64_t tile, uint32_t status, const P& p) {
    uint32_t w[NW] = {};
    __builtin_memcpy(w, &p, sizeof(P));
#pragma unroll
    for (int i = 0; i < NW; i++) st_agent(base + tile * NW + i, ((uint64_t)status << 32) | w[i]);
  }
  // Returns the status (kInvalid when the atoms disagree or are not written yet).
  __device__ static uint32_t load(const uint64_t* base, int64_t tile, P& p) {
    uint32_t w[NW];
    uint32_t st = 0;
    bool same = true;
#pragma unroll
    for (int i = 0; i < NW; i++) {
      uint64_t a = ld_agent(base + tile * NW + i);
      uint32_t s = (uint32_t)(a >> 32);
      w[i] = (uint32_t)a;
      if (i == 0) st = s;
      else same = same && (s == st);
    }
    __builtin_memcpy(&p, w, sizeof(P));
    return same ? st : (uint32_t)kInvalid;
  }
};

// Look-back executed by one full wavefront (all 64 lanes active).  Lane l inspects tile
// `tile - 1 - l`; the window slides back 64 tiles at a time until it contains a tile whose
// inclusive prefix is known.  Returns, in every lane, the reduction of all tiles before
// `tile` in index order:  P[0] (+) P[1] (+) ... (+) P[tile-1]  with a (+) b = f(a, b).
// Tickets are handed out by an atomic counter, so every tile this waits on is already
// running and will publish: the wait is bounded.
template <class P, class F>
__device__ inline P wave_lookback(const uint64_t* desc, int64_t tile, const P id, F f) {
  const int lane = lane_id();
  P prefix = id;
  int64_t pos = tile - 1 - lane;
  while (true) {
    P val = id;
    uint32_t st = kInclusive;  // tiles before tile 0: an empty, fully known prefix
    if (pos >= 0) {
      st = TileDesc<P>::load(desc, pos, val);
      while (st == kInvalid) {
        __builtin_amdgcn_s_sleep(1);
        st = TileDesc<P>::load(desc, pos, val);
      }
    }
    const uint64_t incl = __ballot(st == kInclusive);
    const int first = incl ? __builtin_ctzll(incl) : 64;
    P contrib = (lane <= first) ? val : id;
    // ordered reduction: lane 63 (farthest tile) is leftmost
    P red = wave_inclusive_scan(contrib, id, [&](const P& a, const P& b) { return f(b, a); });
    red = readlane(red, 63);
    prefix = f(red, prefix);
    if (incl) break;
    pos -= 64;
  }
  return prefix;
}

// Look-back for kernels whose tile index is the workgroup index (no ticket).  Nothing then
// guarantees that a tile this waits on has started, so the wait is bounded: a descriptor that is
// still missing after `patience` polls is not waited for any longer — the wavefront computes
// that tile's aggregate itself with aggregate_of(tile_index) (called by all 64 lanes, returns
// the same value in all) and carries on.  Every loop ends whatever the other workgroups do.
// With patience 0 nothing is ever waited for, which is how the tests drive this path.
// aggregate_of reads the tile's INPUT: the caller must not use this when the kernel's output
// may overwrite its input (the owner of a tile that has not published has not written any
// output yet, but it may while the input is being read here); after computing, the descriptor
// is read once more and, if the owner has published meanwhile, its word is taken instead.
template <class P, class F, class A>
__device__ inline P wave_lookback_or_compute(const uint64_t* desc, int64_t tile, const P id, F f, int patience,
                                             A aggregate_of) {
  const int lane = lane_id();
  P prefix = id;
  int64_t nearest = tile - 1;  // lane l inspects tile nearest - l
  while (true) {
    const int64_t pos = nearest - lane;
    P val = id;
    uint32_t st = kInclusive;  // tiles before tile 0: an empty, fully known prefix
    if (pos >= 0) {
      st = TileDesc<P>::load(desc, pos, val);
      for (int polls = 0; st == kInvalid && polls < patience; polls++) {
        __builtin_amdgcn_s_sleep(1);
        st = TileDesc<P>::load(desc, pos, val);
      }
    }
    uint64_t incl = __ballot(st == kInclusive);
    int first = incl ? __builtin_ctzll(incl) : 64;
    uint64_t missing = __ballot(st == kInvalid && lane <= first);  // only tiles that count
    while (missing) {  // wave-uniform
      const int l = __builtin_ctzll(missing);
      missing &= missing - 1;
      const P agg = aggregate_of(nearest - l);
      P now = id;
      const uint32_t st_now = TileDesc<P>::load(desc, nearest - l, now);
      if (lane == l) {
        if (st_now != kInvalid) { val = now; st = st_now; }
        else { val = agg; st = kPartial; }
      }
    }
    incl = __ballot(st == kInclusive);
    first = incl ? __builtin_ctzll(incl) : 64;
    P contrib = (lane <= first) ? val : id;
    // ordered reduction: lane 63 (farthest tile) is leftmost
    P red = wave_inclusive_scan(contrib, id, [&](const P& a, const P& b) { return f(b, a); });
    red = readlane(red, 63);
    prefix = f(red, prefix);
    if (incl) break;
    nearest -= 64;
  }
  return prefix;
}
// Polls of a missing tile descriptor before a ticketless kernel computes it itself (default
// kDefaultLookbackPatience); set by thrust_cdna4_set_lookback_patience.
constexpr int kDefaultLookbackPatience = 256;
int lookback_patience();
// Test knob (thrust_cdna4_set_test_publish_delay): tile 0 of a ticketless kernel sleeps this many
// times (a few microseconds each) before it publishes its descriptor.  0 in normal use.
int lookback_test_publish_delay();
// true when [a, a + na) and [b, b + nb) share a byte
inline bool ranges_overlap(const void* a, size_t na, const void* b, size_t nb) {
  const uintptr_t x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
  return x < y + nb && y < x + na;
}

// ---------------------------------------------------------------------------------------
// Host-side dtype helpers
// ---------------------------------------------------------------------------------------
inline int dtype_size(int dt) {
  switch (dt) {
    case THRUST_CDNA4_I8: case THRUST_CDNA4_U8: return 1;
    case THRUST_CDNA4_I16: case THRUST_CDNA4_U16: return 2;
    case THRUST_CDNA4_I32: case THRUST_CDNA4_U32: case THRUST_CDNA4_F32: return 4;
    case THRUST_CDNA4_I64: case THRUST_CDNA4_U64: case THRUST_CDNA4_F64: return 8;
  }
  return 0;
}

// Calls f(T{}) with the C++ type of `dt`; returns false for an unknown code.
template <class F>
inline bool dispatch_dtype(int dt, F&& f) {
  switch (dt) {
    case THRUST_CDNA4_I8: f(int8_t{}); return true;
    case THRUST_CDNA4_U8: f(uint8_t{}); return true;
    case THRUST_CDNA4_I16: f(int16_t{}); return true;
    case THRUST_CDNA4_U16: f(uint16_t{}); return true;
    case THRUST_CDNA4_I32: f(int32_t{}); return true;
    case THRUST_CDNA4_U32: f(uint32_t{}); return true;
    case THRUST_CDNA4_I64: f(int64_t{}); return true;
    case THRUST_CDNA4_U64: f(uint64_t{}); return true;
    case THRUST_CDNA4_F32: f(float{}); return true;
    case THRUST_CDNA4_F64: f(double{}); return true;
  }
  return false;
}

template <class F>
inline bool dispatch_op(int op, F&& f) {
  switch (op) {
    case THRUST_CDNA4_PLUS: f(OpPlus{}); return true;
    case THRUST_CDNA4_MULTIPLIES: f(OpMultiplies{}); return true;
    case THRUST_CDNA4_MAXIMUM: f(OpMaximum{}); return true;
    case THRUST_CDNA4_MINIMUM: f(OpMinimum{}); return true;
  }
  return false;
}

// Compute units of the current device (cached per device); 256 if the query fails.
int device_cu_count();

// Optional launch profiling: when enabled, every kernel launch of the library is bracketed by
// HIP events on the launch stream and logged under its name (the counterpart of the
// reference's THRUST_DEBUG_SYNC launch log, thrust/system/cuda/detail/core/agent_launcher.h:523-559).
bool profile_enabled();
void profile_begin(const char* name, hipStream_t stream);
void profile_end(hipStream_t stream);

#define TCD_LAUNCH(name, kernel, grid, block, stream, ...)                   \
  do {                                                                       \
    if (::tcd::profile_enabled()) ::tcd::profile_begin(name, stream);        \
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);         \
    if (::tcd::profile_enabled()) ::tcd::profile_end(stream);                \
  } while (0)

// A small zero-fill kernel: used instead of hipMemsetAsync so that every entry point can be
// recorded into a HIP graph.
__global__ void zero_words_kernel(uint32_t* p, size_t nwords);

// The descriptors in a call's temporary storage are 64-bit atoms: an address that is not a multiple
// of 8 would fault on the device, so such a call is refused on the host (the interface asks for 256).
inline bool temp_misaligned(const void* temp) { return (reinterpret_cast<uintptr_t>(temp) & 7u) != 0; }

hipError_t zero_async(void* p, size_t bytes, hipStream_t stream);
// dst[0, bytes) = src[0, bytes) on the device, enqueued on `stream` (non-overlapping ranges)
hipError_t copy_async(void* dst, const void* src, size_t bytes, hipStream_t stream);

}  // namespace tcd
