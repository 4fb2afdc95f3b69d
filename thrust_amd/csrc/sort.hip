// Onesweep least-significant-digit radix sort for gfx950.
//
//   1. radix_hist_kernel   one read of the keys; LDS-privatised 256-bin histograms of ALL
//                          digit places, merged into global memory with atomics.
//   2. radix_bins_kernel   exclusive scan of each digit place's 256 bins.
//   3. onesweep_kernel     one launch per 8-bit digit.  A workgroup takes a tile by ticket,
//                          ranks its keys stably (wave64 ballot "match" ranking on per-wave
//                          LDS counters), publishes its 256 digit counts, finds the counts
//                          of all earlier tiles by decoupled look-back (one thread per
//                          digit), reorders the tile through LDS so that every digit's keys
//                          are contiguous, and writes each run with coalesced stores.
//
// Keys stay in their original representation in memory; the digit is taken from the
// order-preserving encoding of thrust/system/detail/sequential/stable_radix_sort.inl:43-139
// on the fly, so there are no separate encode/decode passes.  Replaces
// thrust/system/cuda/detail/sort.h:213-380 (cub::DeviceRadixSort).
#include "common.h"

namespace tcd {

constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;

// descriptor word: status in bits 31:30, count in bits 29:0
constexpr uint32_t kCountMask = (1u << 30) - 1;

template <int BYTES>
struct uint_of;
template <>
struct uint_of<1> { using type = uint8_t; };
template <>
struct uint_of<2> { using type = uint16_t; };
template <>
struct uint_of<4> { using type = uint32_t; };
template <>
struct uint_of<8> { using type = uint64_t; };

// Order-preserving key encoding on the unsigned bit pattern.  Integer keys: xor with
// `xor_mask` (sign bit for signed types, all ones more for descending order).  Floating
// point: first flip all bits of negatives and the sign bit of non-negatives.
template <class U, bool FLOAT>
__device__ __host__ inline U encode_key(U u, U xor_mask) {
  constexpr int W = 8 * sizeof(U);
  if constexpr (FLOAT) {
    const U sign = U(1) << (W - 1);
    u ^= (u >> (W - 1)) ? U(~U(0)) : sign;
  }
  return u ^ xor_mask;
}
template <class U, bool FLOAT>
__device__ __host__ inline U decode_key(U e, U xor_mask) {
  constexpr int W = 8 * sizeof(U);
  e ^= xor_mask;
  if constexpr (FLOAT) {
    const U sign = U(1) << (W - 1);
    e = (e >> (W - 1)) ? U(e ^ sign) : U(~e);
  }
  return e;
}

// ---------------------------------------------------------------------------------------
// 1. Histogram of every digit place
// ---------------------------------------------------------------------------------------
template <class U, bool FLOAT>
__global__ __launch_bounds__(256) void radix_hist_kernel(const U* __restrict__ keys, int64_t n,
                                                         U xor_mask, uint32_t* ghist, int vec_ok) {
  constexpr int P = sizeof(U);
  constexpr int VEC = 16 / sizeof(U);
  __shared__ uint32_t h[P][kRadix];
  const int tid = threadIdx.x;
#pragma unroll
  for (int p = 0; p < P; p++) h[p][tid] = 0;
  __syncthreads();

  auto count = [&](U k) {
    const U e = encode_key<U, FLOAT>(k, xor_mask);
#pragma unroll
    for (int p = 0; p < P; p++) atomicAdd(&h[p][(uint32_t)(e >> (8 * p)) & 0xffu], 1u);
  };

  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + tid;
  const int64_t gstride = (int64_t)gridDim.x * blockDim.x;
  if (vec_ok) {
    struct alignas(16) V16 { U v[VEC]; };
    const int64_t nvec = n / VEC;
    const V16* kv = reinterpret_cast<const V16*>(keys);
    for (int64_t i = gtid; i < nvec; i += gstride) {
      V16 v = kv[i];
#pragma unroll
      for (int j = 0; j < VEC; j++) count(v.v[j]);
    }
    for (int64_t i = nvec * VEC + gtid; i < n; i += gstride) count(keys[i]);
  } else {
    for (int64_t i = gtid; i < n; i += gstride) count(keys[i]);
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < P; p++) {
    const uint32_t c = h[p][tid];
    if (c) atomicAdd(&ghist[p * kRadix + tid], c);
  }
}

// ---------------------------------------------------------------------------------------
// 2. Exclusive scan of the 256 bins of each digit place (one workgroup per place)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void radix_bins_kernel(uint32_t* ghist) {
  __shared__ uint32_t s_w[4];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  uint32_t* h = ghist + (size_t)blockIdx.x * kRadix;
  const uint32_t c = h[tid];
  uint32_t incl = wave_inclusive_scan(c, 0u, [](uint32_t a, uint32_t b) { return a + b; });
  if (lane == 63) s_w[wave] = incl;
  __syncthreads();
  uint32_t base = 0;
  for (int w = 0; w < wave; w++) base += s_w[w];
  h[tid] = base + incl - c;
}

// ---------------------------------------------------------------------------------------
// 3. One onesweep pass
// ---------------------------------------------------------------------------------------
template <int VB>
struct value_of { using type = typename uint_of<VB>::type; };
template <>
struct value_of<0> { using type = uint32_t; };  // unused placeholder

template <class U, int VB, int BLOCK, int IPT>
struct OnesweepSmem {
  static constexpr int TILE = BLOCK * IPT;
  static constexpr int ELEM = (int)sizeof(U) > VB ? (int)sizeof(U) : VB;
  alignas(16) unsigned char exch[(size_t)TILE * ELEM];  // key / value exchange buffer
  uint32_t wave_cnt[BLOCK / kWave][kRadix];             // per-wave digit counters
  uint32_t local_base[kRadix];                          // first local slot of each digit
  uint32_t global_off[kRadix];                          // global slot of local slot 0, per digit
  uint32_t wave_tot[4];
  uint32_t tile;
};

template <class U, int VB, bool FLOAT, int BLOCK, int IPT>
__global__ __launch_bounds__(BLOCK) void onesweep_kernel(const U* __restrict__ kin, U* __restrict__ kout,
                                                         const void* __restrict__ vin_, void* __restrict__ vout_,
                                                         int64_t n, U xor_mask, int shift,
                                                         const uint32_t* __restrict__ gbase,
                                                         uint32_t* desc, uint32_t* ticket) {
  static_assert(BLOCK % 256 == 0, "one thread per digit needs at least 256 threads");
  using V = typename value_of<VB>::type;
  constexpr int NWAVES = BLOCK / kWave;
  constexpr int TILE = BLOCK * IPT;
  __shared__ OnesweepSmem<U, VB, BLOCK, IPT> sm;
  U* s_keys = reinterpret_cast<U*>(sm.exch);
  V* s_vals = reinterpret_cast<V*>(sm.exch);
  const V* vin = static_cast<const V*>(vin_);
  V* vout = static_cast<V*>(vout_);

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;

  if (tid == 0) sm.tile = atomicAdd(ticket, 1u);
#pragma unroll
  for (int w = 0; w < NWAVES; w++)
    if (tid < kRadix) sm.wave_cnt[w][tid] = 0;
  __syncthreads();
  const int64_t tile = sm.tile;
  const int64_t base = tile * TILE;
  const int valid = (int)((n - base) < (int64_t)TILE ? (n - base) : (int64_t)TILE);

  // ---- load: wave w owns a contiguous slab, item i of lane l is slab[i*64 + l], so the
  //      order (wave, item, lane) is the memory order and ranking in that order is stable.
  const U pad = decode_key<U, FLOAT>(U(~U(0)), xor_mask);  // sorts after every real key
  const int slab = wave * (kWave * IPT) + lane;
  U k[IPT];
#pragma unroll
  for (int i = 0; i < IPT; i++) {
    const int li = slab + i * kWave;
    k[i] = li < valid ? kin[base + li] : pad;
  }

  // ---- rank: for each item, the lanes of this wave holding the same digit (8 ballots),
  //      the count of such lanes below this one, and the wave's running counter.
  volatile uint32_t* wc = sm.wave_cnt[wave];
  const uint64_t lt_mask = (1ull << lane) - 1ull;
  uint32_t pos[IPT];
#pragma unroll
  for (int i = 0; i < IPT; i++) {
    const uint32_t d = (uint32_t)(encode_key<U, FLOAT>(k[i], xor_mask) >> shift) & 0xffu;
    uint64_t m = ~0ull;
#pragma unroll
    for (int b = 0; b < kRadixBits; b++) {
      const bool bit = (d >> b) & 1u;
      const uint64_t bal = __ballot(bit);
      m &= bit ? bal : ~bal;
    }
    const uint32_t below = __popcll(m & lt_mask);
    const uint32_t cnt = __popcll(m);
    const uint32_t old = wc[d];
    if (below == 0) wc[d] = old + cnt;
    pos[i] = old + below;
  }
  __syncthreads();

  // ---- per digit (thread d): exclusive offsets of the waves, tile count, publish, scan
  uint32_t total = 0;
  if (tid < kRadix) {
#pragma unroll
    for (int w = 0; w < NWAVES; w++) {
      const uint32_t c = sm.wave_cnt[w][tid];
      sm.wave_cnt[w][tid] = total;
      total += c;
    }
    const uint32_t st = (tile == 0) ? kInclusive : kPartial;
    st_agent(&desc[tile * kRadix + tid], (st << 30) | total);
    const uint32_t incl = wave_inclusive_scan(total, 0u, [](uint32_t a, uint32_t b) { return a + b; });
    if (lane == 63) sm.wave_tot[wave] = incl;
    sm.local_base[tid] = incl - total;  // completed below
  }
  __syncthreads();
  if (tid < kRadix) {
    uint32_t wbase = 0;
    for (int w = 0; w < wave; w++) wbase += sm.wave_tot[w];
    const uint32_t lbase = sm.local_base[tid] + wbase;
    // look-back over earlier tiles for this digit
    uint32_t prefix = 0;
    if (tile > 0) {
      int64_t t = tile - 1;
      while (true) {
        const uint32_t v = ld_agent(&desc[t * kRadix + tid]);
        const uint32_t st = v >> 30;
        if (st == kInvalid) {
          __builtin_amdgcn_s_sleep(1);
          continue;
        }
        prefix += v & kCountMask;
        if (st == kInclusive) break;
        --t;
      }
      st_agent(&desc[tile * kRadix + tid], ((uint32_t)kInclusive << 30) | (prefix + total));
    }
    sm.global_off[tid] = gbase[tid] + prefix - lbase;
    sm.local_base[tid] = lbase;
  }
  __syncthreads();

  // ---- reorder keys through LDS, then write each digit's run contiguously
#pragma unroll
  for (int i = 0; i < IPT; i++) {
    const uint32_t d = (uint32_t)(encode_key<U, FLOAT>(k[i], xor_mask) >> shift) & 0xffu;
    pos[i] += sm.local_base[d] + sm.wave_cnt[wave][d];
    s_keys[pos[i]] = k[i];
  }
  __syncthreads();
  uint32_t gpos[IPT];
#pragma unroll
  for (int j = 0; j < IPT; j++) {
    const int li = j * BLOCK + tid;
    const U key = s_keys[li];
    const uint32_t d = (uint32_t)(encode_key<U, FLOAT>(key, xor_mask) >> shift) & 0xffu;
    gpos[j] = sm.global_off[d] + (uint32_t)li;
    if (li < valid) kout[gpos[j]] = key;
  }

  if constexpr (VB > 0) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < IPT; i++) {
      const int li = slab + i * kWave;
      V v = V(0);
      if (li < valid) v = vin[base + li];
      s_vals[pos[i]] = v;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < IPT; j++) {
      const int li = j * BLOCK + tid;
      if (li < valid) vout[gpos[j]] = s_vals[li];
    }
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
template <class U, int VB>
struct SortConfig {
  static constexpr int BLOCK = 256;
  static constexpr int IPT = (sizeof(U) + VB > 8) ? 12 : 16;
  static constexpr int TILE = BLOCK * IPT;
};

struct SortPlan {
  size_t keys_alt, vals_alt, hist, tickets, desc, total;
  size_t zero_begin, zero_bytes;
  int64_t ntiles;
};

template <class U, int VB>
static SortPlan make_plan(int64_t n) {
  using C = SortConfig<U, VB>;
  constexpr int P = sizeof(U);
  SortPlan p{};
  p.ntiles = ceil_div(n, C::TILE);
  size_t off = 0;
  p.keys_alt = off; off += align_up((size_t)n * sizeof(U), 256);
  p.vals_alt = off; off += align_up((size_t)n * VB, 256);
  p.zero_begin = off;
  p.hist = off; off += align_up((size_t)P * kRadix * 4, 256);
  p.tickets = off; off += 256;
  p.desc = off; off += align_up((size_t)P * p.ntiles * kRadix * 4, 256);
  p.zero_bytes = off - p.zero_begin;
  p.total = off;
  return p;
}

template <class U, int VB, bool FLOAT>
static hipError_t sort_typed(void* temp, size_t* temp_bytes, void* keys, void* values, int64_t n,
                             U xor_mask, hipStream_t stream) {
  using C = SortConfig<U, VB>;
  constexpr int P = sizeof(U);
  const SortPlan plan = make_plan<U, VB>(n);
  if (temp == nullptr) {
    *temp_bytes = plan.total;
    return hipSuccess;
  }
  if (*temp_bytes < plan.total) return hipErrorInvalidValue;
  if (n == 0) return hipSuccess;
  char* t = static_cast<char*>(temp);
  U* kbuf[2] = {static_cast<U*>(keys), reinterpret_cast<U*>(t + plan.keys_alt)};
  char* vbuf[2] = {static_cast<char*>(values), t + plan.vals_alt};
  uint32_t* ghist = reinterpret_cast<uint32_t*>(t + plan.hist);
  uint32_t* tickets = reinterpret_cast<uint32_t*>(t + plan.tickets);
  uint32_t* desc = reinterpret_cast<uint32_t*>(t + plan.desc);

  hipError_t e = zero_async(t + plan.zero_begin, plan.zero_bytes, stream);
  if (e != hipSuccess) return e;

  const int vec_ok = (reinterpret_cast<uintptr_t>(keys) & 15) == 0;
  int64_t hblocks = ceil_div(n, 256 * 64);
  if (hblocks > 2048) hblocks = 2048;
  TCD_LAUNCH("radix_hist_kernel", (radix_hist_kernel<U, FLOAT>), dim3((unsigned)hblocks), dim3(256), stream,
             kbuf[0], n, xor_mask, ghist, vec_ok);
  TCD_LAUNCH("radix_bins_kernel", radix_bins_kernel, dim3(P), dim3(256), stream, ghist);
  int cur = 0;
  for (int p = 0; p < P; p++) {
    TCD_LAUNCH("onesweep_kernel", (onesweep_kernel<U, VB, FLOAT, C::BLOCK, C::IPT>), dim3((unsigned)plan.ntiles),
               dim3(C::BLOCK), stream, kbuf[cur], kbuf[cur ^ 1], vbuf[cur], vbuf[cur ^ 1], n, xor_mask, 8 * p,
               ghist + p * kRadix, desc + (size_t)p * plan.ntiles * kRadix, tickets + p);
    cur ^= 1;
  }
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (cur == 1) {  // odd number of passes: bring the result home
    e = hipMemcpyAsync(kbuf[0], kbuf[1], (size_t)n * sizeof(U), hipMemcpyDeviceToDevice, stream);
    if (e != hipSuccess) return e;
    if (VB) e = hipMemcpyAsync(vbuf[0], vbuf[1], (size_t)n * VB, hipMemcpyDeviceToDevice, stream);
  }
  return e;
}

template <int VB>
static hipError_t sort_dispatch(void* temp, size_t* temp_bytes, int key_dtype, void* keys, void* values,
                                int64_t n, int descending, hipStream_t s) {
  const bool is_signed = key_dtype == THRUST_CDNA4_I8 || key_dtype == THRUST_CDNA4_I16 ||
                         key_dtype == THRUST_CDNA4_I32 || key_dtype == THRUST_CDNA4_I64;
  auto mask = [&](auto u) {
    using U = decltype(u);
    U m = is_signed ? U(U(1) << (8 * sizeof(U) - 1)) : U(0);
    if (descending) m = U(~m);
    return m;
  };
  switch (key_dtype) {
    case THRUST_CDNA4_I8: case THRUST_CDNA4_U8:
      return sort_typed<uint8_t, VB, false>(temp, temp_bytes, keys, values, n, mask(uint8_t{}), s);
    case THRUST_CDNA4_I16: case THRUST_CDNA4_U16:
      return sort_typed<uint16_t, VB, false>(temp, temp_bytes, keys, values, n, mask(uint16_t{}), s);
    case THRUST_CDNA4_I32: case THRUST_CDNA4_U32:
      return sort_typed<uint32_t, VB, false>(temp, temp_bytes, keys, values, n, mask(uint32_t{}), s);
    case THRUST_CDNA4_I64: case THRUST_CDNA4_U64:
      return sort_typed<uint64_t, VB, false>(temp, temp_bytes, keys, values, n, mask(uint64_t{}), s);
    case THRUST_CDNA4_F32:
      return sort_typed<uint32_t, VB, true>(temp, temp_bytes, keys, values, n, mask(uint32_t{}), s);
    case THRUST_CDNA4_F64:
      return sort_typed<uint64_t, VB, true>(temp, temp_bytes, keys, values, n, mask(uint64_t{}), s);
  }
  return hipErrorInvalidValue;
}

}  // namespace tcd

extern "C" int thrust_cdna4_sort_keys(void* temp, size_t* temp_bytes, int key_dtype, void* keys,
                                      int64_t n, int descending, void* stream) {
  if (!temp_bytes || n < 0 || n >= ((int64_t)1 << 30) || (n > 0 && temp && !keys))
    return hipErrorInvalidValue;
  return (int)tcd::sort_dispatch<0>(temp, temp_bytes, key_dtype, keys, nullptr, n, descending,
                                    static_cast<hipStream_t>(stream));
}

extern "C" int thrust_cdna4_sort_pairs(void* temp, size_t* temp_bytes, int key_dtype, void* keys,
                                       int value_bytes, void* values, int64_t n, int descending,
                                       void* stream) {
  if (!temp_bytes || n < 0 || n >= ((int64_t)1 << 30) || (n > 0 && temp && (!keys || !values)))
    return hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (value_bytes) {
    case 1: return (int)tcd::sort_dispatch<1>(temp, temp_bytes, key_dtype, keys, values, n, descending, s);
    case 2: return (int)tcd::sort_dispatch<2>(temp, temp_bytes, key_dtype, keys, values, n, descending, s);
    case 4: return (int)tcd::sort_dispatch<4>(temp, temp_bytes, key_dtype, keys, values, n, descending, s);
    case 8: return (int)tcd::sort_dispatch<8>(temp, temp_bytes, key_dtype, keys, values, n, descending, s);
  }
  return hipErrorInvalidValue;
}
