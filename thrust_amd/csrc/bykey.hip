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

namespace tcd {

template <int B> struct key_bits;
template <> struct key_bits<1> { using type = uint8_t; };
template <> struct key_bits<2> { using type = uint16_t; };
template <> struct key_bits<4> { using type = uint32_t; };
template <> struct key_bits<8> { using type = uint64_t; };
using KU = key_bits<TCD_KEY_BYTES>::type;

template <class T>
struct SegPair {
  uint32_t c;  // heads seen
  T v;         // value of the open segment
};

template <class T, class Op>
__device__ inline SegPair<T> seg_combine(const SegPair<T>& a, const SegPair<T>& b) {
  SegPair<T> r;
  r.c = a.c + b.c;
  r.v = b.c ? b.v : Op::template apply<T>(a.v, b.v);
  return r;
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

template <int N, class E>
struct alignas(N * sizeof(E)) VecN {
  E v[N];
};

// Geometry shared by both kernels: a thread owns VEC consecutive elements of each of
// CHUNKS chunks; VEC is set by the wider of key and value so that no access exceeds 16 B.
template <class T>
struct SegGeom {
#ifndef TCD_SEG_BLOCK
#define TCD_SEG_BLOCK 256
#define TCD_SEG_CHUNKS 4
#endif
  static constexpr int BLOCK = TCD_SEG_BLOCK;
  static constexpr int WIDE = (int)(sizeof(KU) > sizeof(T) ? sizeof(KU) : sizeof(T));
  static constexpr int VEC = 16 / WIDE;
  static constexpr int CHUNKS = WIDE >= 4 ? TCD_SEG_CHUNKS : 2;
  static constexpr int NWAVES = BLOCK / kWave;
  static constexpr int64_t TILE = (int64_t)BLOCK * VEC * CHUNKS;
};

// Loads a tile, computes head flags, scans it and resolves the tile prefix by look-back.
// On return: key/val/head hold the thread's elements, incl[c][j] the segmented inclusive
// pair of element (c, j) counted from the start of the thread's group, and off[c] the pair
// of everything before the group (all earlier tiles included).
template <class T, class Op>
struct SegTile {
  using G = SegGeom<T>;
  using Pair = SegPair<T>;
  static constexpr int VEC = G::VEC, CHUNKS = G::CHUNKS, NWAVES = G::NWAVES, BLOCK = G::BLOCK;

  struct Smem {
    Pair tot[CHUNKS][NWAVES];
    Pair prefix;
    uint32_t tile;
  };

  KU key[CHUNKS][VEC];
  T val[CHUNKS][VEC];
  bool head[CHUNKS][VEC];
  Pair incl[CHUNKS][VEC];
  Pair off[CHUNKS];
  int64_t base;
  int64_t tile;

  __device__ int64_t index(int c, int j) const {
    return base + ((int64_t)c * BLOCK + threadIdx.x) * VEC + j;
  }

  __device__ void run(Smem& sm, const KU* keys, const T* vals, int64_t n, int float_keys, int vec_ok,
                      uint64_t* desc, uint32_t* ticket) {
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const T id = Op::template identity<T>();
    const Pair idp{0u, id};
    auto comb = [](const Pair& a, const Pair& b) { return seg_combine<T, Op>(a, b); };

    if (tid == 0) sm.tile = atomicAdd(ticket, 1u);
    __syncthreads();
    tile = sm.tile;
    base = tile * G::TILE;
    const bool fast = vec_ok && (base + G::TILE <= n);

#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      const int64_t i0 = index(c, 0);
      KU prev = 0;
      if (i0 > 0 && i0 < n) prev = keys[i0 - 1];
      if (fast) {
        const auto kv = *reinterpret_cast<const VecN<VEC, KU>*>(keys + i0);
        const auto vv = *reinterpret_cast<const VecN<VEC, T>*>(vals + i0);
#pragma unroll
        for (int j = 0; j < VEC; j++) { key[c][j] = kv.v[j]; val[c][j] = vv.v[j]; }
      } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) {
          const int64_t idx = i0 + j;
          key[c][j] = idx < n ? keys[idx] : KU(0);
          val[c][j] = idx < n ? vals[idx] : id;
        }
      }
#pragma unroll
      for (int j = 0; j < VEC; j++) {
        const int64_t idx = i0 + j;
        const KU p = j == 0 ? prev : key[c][j - 1];
        head[c][j] = idx < n && (idx == 0 || keys_differ(p, key[c][j], float_keys));
      }
    }

    Pair excl_w[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      incl[c][0] = Pair{head[c][0] ? 1u : 0u, val[c][0]};
#pragma unroll
      for (int j = 1; j < VEC; j++) incl[c][j] = comb(incl[c][j - 1], Pair{head[c][j] ? 1u : 0u, val[c][j]});
      const Pair w = wave_inclusive_scan(incl[c][VEC - 1], idp, comb);
      excl_w[c] = wave_shift_up1(w, idp);
      if (lane == kWave - 1) sm.tot[c][wave] = w;
    }
    __syncthreads();

    Pair seg_base[CHUNKS];
    Pair run = idp;
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
#pragma unroll
      for (int w = 0; w < NWAVES; w++) {
        if (w == wave) seg_base[c] = run;
        run = comb(run, sm.tot[c][w]);
      }
    }
    const Pair tile_agg = run;

    if (wave == 0) {
      Pair prefix = idp;
      if (tile == 0) {
        if (lane == 0) TileDesc<Pair>::store(desc, 0, kInclusive, tile_agg);
      } else {
        if (lane == 0) TileDesc<Pair>::store(desc, tile, kPartial, tile_agg);
        prefix = wave_lookback<Pair>(desc, tile, idp, comb);
        if (lane == 0) TileDesc<Pair>::store(desc, tile, kInclusive, comb(prefix, tile_agg));
      }
      if (lane == 0) sm.prefix = prefix;
    }
    __syncthreads();
    const Pair prefix = sm.prefix;
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) off[c] = comb(comb(prefix, seg_base[c]), excl_w[c]);
  }
};

// ---------------------------------------------------------------------------------------
// scan_by_key
// ---------------------------------------------------------------------------------------
template <class T, class Op>
__global__ __launch_bounds__(SegGeom<T>::BLOCK) void scan_by_key_kernel(
    const KU* keys, const T* vals, T* out, int64_t n, T init, int exclusive, int float_keys, int vec_ok,
    uint64_t* desc, uint32_t* ticket) {
  using ST = SegTile<T, Op>;
  __shared__ typename ST::Smem sm;
  ST t;
  t.run(sm, keys, vals, n, float_keys, vec_ok, desc, ticket);
  constexpr int VEC = ST::VEC, CHUNKS = ST::CHUNKS;
  const bool fast = vec_ok && (t.base + SegGeom<T>::TILE <= n);
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    T r[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      if (!exclusive) {
        r[j] = seg_combine<T, Op>(t.off[c], t.incl[c][j]).v;
      } else {
        // value of the open segment just before this element
        const T before = j == 0 ? t.off[c].v : seg_combine<T, Op>(t.off[c], t.incl[c][j - 1]).v;
        r[j] = t.head[c][j] ? init : Op::template apply<T>(init, before);
      }
    }
    const int64_t i0 = t.index(c, 0);
    if (fast) {
      VecN<VEC, T> v;
#pragma unroll
      for (int j = 0; j < VEC; j++) v.v[j] = r[j];
      *reinterpret_cast<VecN<VEC, T>*>(out + i0) = v;
    } else {
#pragma unroll
      for (int j = 0; j < VEC; j++)
        if (i0 + j < n) out[i0 + j] = r[j];
    }
  }
}

// ---------------------------------------------------------------------------------------
// reduce_by_key
// ---------------------------------------------------------------------------------------
template <class T, class Op>
__global__ __launch_bounds__(SegGeom<T>::BLOCK) void reduce_by_key_kernel(
    const KU* keys, const T* vals, KU* keys_out, T* vals_out, int64_t* num_runs, int64_t n,
    int float_keys, int vec_ok, uint64_t* desc, uint32_t* ticket) {
  using ST = SegTile<T, Op>;
  __shared__ typename ST::Smem sm;
  ST t;
  t.run(sm, keys, vals, n, float_keys, vec_ok, desc, ticket);
  constexpr int VEC = ST::VEC, CHUNKS = ST::CHUNKS;
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
#pragma unroll
    for (int j = 0; j < VEC; j++) {
      const int64_t idx = t.index(c, j);
      if (idx >= n) continue;
      // pair of everything before this element: (runs started so far, value of the open run)
      const SegPair<T> before = j == 0 ? t.off[c] : seg_combine<T, Op>(t.off[c], t.incl[c][j - 1]);
      if (t.head[c][j]) {
        keys_out[before.c] = t.key[c][j];
        if (idx > 0) vals_out[before.c - 1] = before.v;
      }
      if (idx == n - 1) {
        const SegPair<T> last = seg_combine<T, Op>(t.off[c], t.incl[c][j]);
        vals_out[last.c - 1] = last.v;
        *num_runs = (int64_t)last.c;
      }
    }
  }
}

template <class T>
static size_t bykey_temp_bytes(int64_t n) {
  const int64_t ntiles = ceil_div(n, SegGeom<T>::TILE);
  return 256 + align_up((size_t)ntiles * TileDesc<SegPair<T>>::kBytesPerTile, 256);
}

#define TCD_CAT2(a, b) a##b
#define TCD_CAT(a, b) TCD_CAT2(a, b)

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
      const size_t need = bykey_temp_bytes<T>(n);
      if (!temp) { *temp_bytes = need; rc = hipSuccess; return; }
      if (*temp_bytes < need) return;
      if (n == 0) { rc = hipSuccess; return; }
      rc = zero_async(temp, need, s);
      if (rc != hipSuccess) return;
      T iv = T(0);
      if (init) __builtin_memcpy(&iv, init, sizeof(T));
      const int vec_ok = ((reinterpret_cast<uintptr_t>(keys) | reinterpret_cast<uintptr_t>(values) |
                           reinterpret_cast<uintptr_t>(out)) & 15) == 0;
      const int64_t ntiles = ceil_div(n, SegGeom<T>::TILE);
      TCD_LAUNCH("scan_by_key_kernel", (scan_by_key_kernel<T, Op>), dim3((unsigned)ntiles), dim3(SegGeom<T>::BLOCK), s,
                         static_cast<const KU*>(keys), static_cast<const T*>(values), static_cast<T*>(out),
                         n, iv, exclusive, float_keys, vec_ok,
                         reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256),
                         reinterpret_cast<uint32_t*>(temp));
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
      const size_t need = bykey_temp_bytes<T>(n);
      if (!temp) { *temp_bytes = need; rc = hipSuccess; return; }
      if (*temp_bytes < need) return;
      if (n == 0) {  // no runs: only the count is written
        rc = zero_async(num_runs_out, sizeof(int64_t), s);
        return;
      }
      rc = zero_async(temp, need, s);
      if (rc != hipSuccess) return;
      const int vec_ok = ((reinterpret_cast<uintptr_t>(keys_in) | reinterpret_cast<uintptr_t>(values_in)) & 15) == 0;
      const int64_t ntiles = ceil_div(n, SegGeom<T>::TILE);
      TCD_LAUNCH("reduce_by_key_kernel", (reduce_by_key_kernel<T, Op>), dim3((unsigned)ntiles), dim3(SegGeom<T>::BLOCK), s,
                         static_cast<const KU*>(keys_in), static_cast<const T*>(values_in),
                         static_cast<KU*>(keys_out), static_cast<T*>(values_out), num_runs_out, n, float_keys,
                         vec_ok, reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + 256),
                         reinterpret_cast<uint32_t*>(temp));
      rc = hipGetLastError();
    });
  });
  return (int)rc;
}
