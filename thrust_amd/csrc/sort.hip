// Onesweep least-significant-digit radix sort for gfx950.
//
//   1. radix_hist_kernel   one read of the keys; LDS-privatised 256-bin histograms of ALL
//                          digit places (replicated per lane), merged into global memory
//                          with atomics.  It also clears the passes' tile descriptors.
//   2. radix_bins          exclusive scan of each digit place's 256 bins and the choice of the
//                          passes that run, by the histogram kernel's last workgroup.
//   3. onesweep_kernel     one launch per 8-bit digit.  A workgroup takes a tile by ticket,
//                          ranks its keys stably (returning LDS atomics on per-wave digit
//                          counters), publishes its 256 digit counts, finds the counts
//                          of all earlier tiles by decoupled look-back (one thread per
//                          digit), reorders the tile through LDS so that every digit's keys
//                          are contiguous, and writes each run with coalesced stores.
//
// Stability of the ranking rests on one property of the LDS unit: the lanes of one wavefront
// instruction that add to the same LDS address receive their old values in lane order.
// thrust_cdna4_selftest_lds_atomic_order() (below) checks it on the device at hand.
//
// Keys stay in their original representation in memory; the digit is taken from the
// order-preserving encoding of thrust/system/detail/sequential/stable_radix_sort.inl:43-139
// on the fly, so there are no separate encode/decode passes.  Replaces
// thrust/system/cuda/detail/sort.h:213-380 (cub::DeviceRadixSort).
#include <atomic>
#include <mutex>

#include <vector>

#include "common.h"

namespace tcd {

constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;

// Descriptor word D (uint32_t for n < 2^30, uint64_t up to the limit of 32-bit positions):
// status in the two top bits, count below.
template <class D>
struct DescWord {
  static constexpr int kShift = 8 * (int)sizeof(D) - 2;
  static constexpr D kCountMask = (D(1) << kShift) - 1;
  __device__ static D make(uint32_t status, uint32_t count) { return (D(status) << kShift) | D(count); }
  __device__ static uint32_t status(D w) { return (uint32_t)(w >> kShift); }
  __device__ static uint32_t count(D w) { return (uint32_t)(w & kCountMask); }
};
constexpr int kLookW = 8;  // look-back descriptors loaded per round trip
// Consecutive tiles write the ends of their per-digit runs into the same cache lines.  Groups of
// this many consecutive tiles are processed by one XCD, so that seven of eight such lines are put
// together in that XCD's L2 instead of being written to memory in two pieces (see take_tile).
constexpr int kXcdGroup = 8;
constexpr int kXcds = 8;             // the scheme is used on devices that spread workgroup i to XCD i mod 8
constexpr int kXcdCounterStride = 32;  // words: each XCD's counter in a cache line of its own

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
// 2. Exclusive scan of the 256 bins of each digit place, and which passes run
// ---------------------------------------------------------------------------------------
// Run by ONE workgroup of at least 256 threads — the histogram kernel's workgroup that finishes
// last (below) — for all P places; it then decides which passes run.  A place where every
// key has the same digit is the identity permutation for a stable sort, so its pass is skipped
// (64-bit keys that hold small numbers, keys with constant fields, all-equal keys).  The number of
// passes that run is kept even, so that the result ends in the caller's buffer without a copy: if
// an odd number of places need their pass, one of the skippable ones runs as well.  The decision
// travels in the pass's ticket counter, which every workgroup of the pass reads anyway: the
// counter starts at kPassSkipped for a pass that does not run and at kPassReadsAlt for one whose
// input is the alternate buffer; the tile number is in the low bits.  With skipping off every
// pass runs (places = 1: the caller copies the result back).
// The counts are read with agent-scope loads: the other workgroups added them with agent-scope
// atomics, possibly from another XCD, and this workgroup's L2 must not answer from an older line.
constexpr uint32_t kPassSkipped = 0x80000000u, kPassReadsAlt = 0x40000000u, kTicketMask = 0x3FFFFFFFu;
__device__ inline void radix_bins(uint32_t* ghist, int places, uint32_t n, uint32_t* tickets, int skipping) {
  __shared__ uint32_t s_w[4];
  __shared__ uint32_t s_same[8];  // places is at most 8
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const bool mine = tid < kRadix;  // thread d has digit d; the others only keep the barriers' count
  if (tid < 8) s_same[tid] = 0;
  for (int p = 0; p < places; p++) {
    __syncthreads();
    uint32_t* h = ghist + (size_t)p * kRadix;
    const uint32_t c = mine ? ld_agent(&h[tid]) : 0u;
    if (mine && c == n) s_same[p] = 1;  // all keys in one bin
    uint32_t incl = wave_inclusive_scan(c, 0u, [](uint32_t a, uint32_t b) { return a + b; });
    if (mine && lane == 63) s_w[wave] = incl;
    __syncthreads();
    uint32_t base = 0;
    for (int w = 0; w < wave && w < 4; w++) base += s_w[w];
    if (mine) h[tid] = base + incl - c;
  }
  __syncthreads();
  if (tid == 0) {
    int needed = 0;
    for (int p = 0; p < places; p++) needed += s_same[p] ? 0 : 1;
    bool one_more = skipping && (needed & 1);  // keep the number of passes even
    uint32_t reads_alt = 0;
    for (int p = 0; p < places; p++) {
      bool runs = !skipping || !s_same[p];
      if (!runs && one_more) {
        runs = true;
        one_more = false;
      }
      tickets[p] = runs ? reads_alt : kPassSkipped;
      if (runs) reads_alt ^= kPassReadsAlt;
    }
  }
}

// ---------------------------------------------------------------------------------------
// 1. Histogram of every digit place (and, in its last workgroup, step 2)
// ---------------------------------------------------------------------------------------
// Counters are replicated per lane: the counter of (place, digit, copy) lives at word
// (place*256 + digit)*COPIES + copy with copy = lane % COPIES, so the lanes of a wave spread
// over the LDS banks whatever the keys are (random, sorted, constant) instead of meeting on
// the few banks their digits select.  64 KiB per workgroup: 16 copies for 4-byte keys, 8 for
// 8-byte keys, 32 for narrower ones.
constexpr int kHistThreads = 512;
template <class U>
struct RadixHistGeom {
  static constexpr int P = sizeof(U);
  static constexpr int COPIES = 16384 / (P * kRadix) > 32 ? 32 : 16384 / (P * kRadix);
};

// The kernel also clears the tile descriptors of the passes that follow (`clear`, `clear_bytes`:
// a multiple of 16).  Nothing reads them before the first pass starts, the stores need no answer
// and go out under the key loads, and the clearing launch in front of this kernel is left with the
// few KiB that must be zero before the first count arrives (status, histogram, tickets).
template <class U, bool FLOAT>
__global__ __launch_bounds__(kHistThreads) void radix_hist_kernel(const U* __restrict__ keys, int64_t n,
                                                                  U xor_mask, uint32_t* ghist, int vec_ok,
                                                                  void* clear, size_t clear_bytes,
                                                                  uint32_t* tickets, uint32_t* done, int skipping) {
  constexpr int P = RadixHistGeom<U>::P;
  constexpr int COPIES = RadixHistGeom<U>::COPIES;
  constexpr int VEC = 16 / sizeof(U);
  constexpr int UNROLL = 8;  // 128-bit loads in flight per thread
  __shared__ uint32_t h[P * kRadix * COPIES];
  const int tid = threadIdx.x;
  {
    const size_t first = (size_t)blockIdx.x * kHistThreads + tid, step = (size_t)gridDim.x * kHistThreads;
    if ((reinterpret_cast<uintptr_t>(clear) & 15u) == 0) {
      tcd_v4u* c16 = static_cast<tcd_v4u*>(clear);
      for (size_t i = first; i < clear_bytes / 16; i += step) c16[i] = tcd_v4u{0u, 0u, 0u, 0u};
    } else {  // temporary storage that is not aligned as asked for: words
      uint32_t* c4 = static_cast<uint32_t*>(clear);
      for (size_t i = first; i < clear_bytes / 4; i += step) c4[i] = 0u;
    }
  }
  for (int i = tid; i < P * kRadix * COPIES; i += kHistThreads) h[i] = 0;
  __syncthreads();

  uint32_t* mine = h + (tid & (COPIES - 1));
  auto count = [&](U k) {
    const U e = encode_key<U, FLOAT>(k, xor_mask);
#pragma unroll
    for (int p = 0; p < P; p++) {
      const uint32_t d = (uint32_t)(e >> (8 * p)) & 0xffu;
      atomicAdd(mine + (p * kRadix + d) * COPIES, 1u);
    }
  };

  const int64_t gtid = (int64_t)blockIdx.x * kHistThreads + tid;
  const int64_t gstride = (int64_t)gridDim.x * kHistThreads;
  if (vec_ok) {
    struct alignas(16) V16 { U v[VEC]; };
    const int64_t nvec = n / VEC;
    const V16* kv = reinterpret_cast<const V16*>(keys);
    int64_t i = gtid;
    for (; i + (UNROLL - 1) * gstride < nvec; i += UNROLL * gstride) {
      V16 v[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; u++) v[u] = load16<V16>(&kv[i + u * gstride]);
#pragma unroll
      for (int u = 0; u < UNROLL; u++)
#pragma unroll
        for (int j = 0; j < VEC; j++) count(v[u].v[j]);
    }
    for (; i < nvec; i += gstride) {
      const V16 v = load16<V16>(&kv[i]);
#pragma unroll
      for (int j = 0; j < VEC; j++) count(v.v[j]);
    }
    for (int64_t r = nvec * VEC + gtid; r < n; r += gstride) count(keys[r]);
  } else {
    for (int64_t r = gtid; r < n; r += gstride) count(keys[r]);
  }
  __syncthreads();
  for (int b = tid; b < P * kRadix; b += kHistThreads) {
    uint32_t c = 0;
#pragma unroll
    for (int r = 0; r < COPIES; r++) c += h[b * COPIES + ((r + b) & (COPIES - 1))];  // rotated: spread over banks
    if (c) atomicAdd(&ghist[b], c);
  }
  // The workgroup that finishes last scans the bins: every thread's counts are out (fence) before
  // its workgroup is counted as done, and the one that counts the last sees them all (fence).
  // `done` starts at zero like the histogram.
  __shared__ uint32_t s_last;
  __threadfence();
  __syncthreads();
  if (tid == 0) s_last = atomicAdd(done, 1u) == gridDim.x - 1u ? 1u : 0u;
  __syncthreads();
  if (s_last == 0u) return;
  __threadfence();
  radix_bins(ghist, P, (uint32_t)n, tickets, skipping);
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
  uint16_t wave_cnt[BLOCK / kWave][kRadix];             // per-wave digit counts (two per LDS word), then first local slots
  uint32_t global_off[kRadix];                          // global slot of local slot 0, per digit
  uint32_t wave_tot[4];
  uint32_t tile;
};

__device__ inline uint32_t lds_load(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
}
__device__ inline void lds_store(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
}

// Look-back polls that find nothing new before a digit's thread gives up (seconds: far beyond
// any wait that ends).  The kernel then still runs to completion, with wrong positions that
// stay inside the output; the event is recorded in the status word of the sort call (the first
// word of its temporary storage, read by thrust_cdna4_sort_status) and counted per device in
// g_lookback_timeouts.
constexpr uint32_t kLookbackSpinLimit = 1u << 22;
__device__ unsigned int g_lookback_timeouts;
__device__ inline void note_timeout(uint32_t* status) {
  atomicOr(status, 1u);
  atomicAdd(&g_lookback_timeouts, 1u);
}

// The tile a workgroup processes, with the pass's flags in the top bits.  Plain form (xcd == nullptr):
// the next ticket of the pass's counter — tiles start in index order, so every tile that a look-back
// waits for is running.  Grouped form: workgroup i runs on XCD i mod 8 (checked on the device before
// this form is used); the workgroups of an XCD take the tiles of the XCD's current group of kXcdGroup
// consecutive tiles in order, and the one that takes the first tile of a group claims the group from
// the pass's counter and leaves its number for the others.  An XCD's tiles are still started in index
// order and groups are claimed in index order, so the lowest tile that has not started belongs to an
// XCD all of whose running tiles are lower — they need nothing from it and finish —, and that XCD
// starts its next workgroup whatever the other XCDs are doing (also checked): every wait ends.
__device__ inline uint32_t take_tile(uint32_t* ticket, uint32_t* xcd, int xcd_slots, uint32_t spin_limit, uint32_t* status) {
  if (xcd == nullptr) return atomicAdd(ticket, 1u);
  const uint32_t x = blockIdx.x % kXcds;
  const uint32_t idx = atomicAdd(&xcd[x * kXcdCounterStride], 1u);
  const uint32_t slot = idx / kXcdGroup, within = idx % kXcdGroup;
  uint32_t* cell = &xcd[kXcds * kXcdCounterStride + x * xcd_slots + slot];
  uint32_t group_word;
  if (within == 0) {
    group_word = atomicAdd(ticket, 1u);
    st_agent(cell, group_word + 1u);  // never 0: the cell starts at 0
  } else {
    // the workgroup that took the group's first tile started before this one and writes the cell
    // right after its own atomic; the poll limit only makes sure that the loop ends
    uint32_t v = ld_agent(cell), spins = 0;
    while (v == 0u && ++spins < spin_limit) {
      __builtin_amdgcn_s_sleep(1);
      v = ld_agent(cell);
    }
    if (v == 0u) {
      // no group number: the workgroup leaves (as for a skipped pass); the tile it would have
      // taken is never published, the tiles after it time out as well, and the call reports it
      note_timeout(status);
      return kPassSkipped;
    }
    group_word = v - 1u;
  }
  return (group_word & ~kTicketMask) | ((group_word & kTicketMask) * kXcdGroup + within);
}

template <class U, int VB, bool FLOAT, int BLOCK, int IPT, int WPE, class D>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(WPE))) void onesweep_kernel(U* kmain, U* kalt, void* vmain, void* valt,
                                                         int64_t n, U xor_mask, int shift,
                                                         const uint32_t* __restrict__ gbase,
                                                         D* desc, uint32_t* ticket, uint32_t* xcd, int xcd_slots,
                                                         uint32_t* status, uint32_t spin_limit, int publish_delay) {
  static_assert(BLOCK % 256 == 0, "one thread per digit needs at least 256 threads");
  using V = typename value_of<VB>::type;
  constexpr int NWAVES = BLOCK / kWave;
  constexpr int TILE = BLOCK * IPT;
  __shared__ OnesweepSmem<U, VB, BLOCK, IPT> sm;
  U* s_keys = reinterpret_cast<U*>(sm.exch);
  V* s_vals = reinterpret_cast<V*>(sm.exch);
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;

  if (tid == 0) sm.tile = take_tile(ticket, xcd, xcd_slots, spin_limit, status);
  if (tid < kRadix / 2) {
#pragma unroll
    for (int w = 0; w < NWAVES; w++) reinterpret_cast<uint32_t*>(sm.wave_cnt[w])[tid] = 0;
  }
  __syncthreads();
  const uint32_t ticket_word = sm.tile;  // tile number, and what radix_bins decided about this pass
  if (ticket_word & kPassSkipped) return;  // every key has the same digit here
  const bool from_alt = (ticket_word & kPassReadsAlt) != 0;
  const U* __restrict__ kin = from_alt ? kalt : kmain;
  U* __restrict__ kout = from_alt ? kmain : kalt;
  const V* __restrict__ vin = static_cast<const V*>(from_alt ? valt : vmain);
  V* __restrict__ vout = static_cast<V*>(from_alt ? vmain : valt);
  const int64_t tile = ticket_word & kTicketMask;
  if (tile * TILE >= n) return;  // a workgroup of the padding that makes every XCD's share whole groups
  const int64_t base = tile * TILE;
  const int valid = (int)((n - base) < (int64_t)TILE ? (n - base) : (int64_t)TILE);
  const bool full = valid == TILE;

  // registers and the LDS exchange buffer hold ENCODED keys (one copy per key); the original
  // bit pattern is restored when a key is written back to global memory
  auto digit_of = [&](U enc) -> uint32_t { return (uint32_t)(enc >> shift) & 0xffu; };

  // ---- load: wave w owns a contiguous slab, item i of lane l is slab[i*64 + l], so the
  //      order (wave, item, lane) is the memory order and ranking in that order is stable.
  const int slab = wave * (kWave * IPT) + lane;
  U k[IPT];
  if (full) {
#pragma unroll
    for (int i = 0; i < IPT; i++) k[i] = encode_key<U, FLOAT>(kin[base + slab + i * kWave], xor_mask);
  } else {
#pragma unroll
    for (int i = 0; i < IPT; i++) {
      // every lane loads (the last valid key where it has none of its own): a load under a
      // per-item branch would wait for the one before it
      const int li = slab + i * kWave;
      const U got = encode_key<U, FLOAT>(kin[base + (li < valid ? li : valid - 1)], xor_mask);
      k[i] = li < valid ? got : U(~U(0));  // padding sorts last
    }
  }

  // ---- rank within (wave, digit): the value returned by the wave's LDS atomic add.  The LDS
  //      unit serves the lanes of one instruction that hit the same address in lane order, so
  //      the returned values number a digit's keys in (item, lane) order, which is the memory
  //      order of the wave's slab: the ranking is stable.  Afterwards the counters hold the
  //      per-wave digit counts, published before the reorder so that later tiles rarely wait.
  // Counters are 16 bits wide (a wave holds at most 64*IPT keys), two digits per LDS word: the
  // atomic adds 1 to the half of the key's digit and the rank is that half of the old value.
  // Ranks are kept two per register until the reorder.
  static_assert(kWave * IPT < 65536 && TILE < 65536, "16-bit counters and local slots");
  uint32_t* wc = reinterpret_cast<uint32_t*>(sm.wave_cnt[wave]);
  const uint16_t* wc16 = sm.wave_cnt[wave];
  uint32_t rk[(IPT + 1) / 2];
  auto keep_rank = [&](int i, uint32_t old, uint32_t sh) {
    const uint32_t r = (old >> sh) & 0xffffu;
    if (i & 1) rk[i / 2] |= r << 16;
    else rk[i / 2] = r;
  };
  {
    // A wave whose 64 keys share one digit (sorted or low-entropy input) would serialise 64
    // same-address atomics.  The first item decides which loop the wave runs (random keys pay
    // for no test at all); the careful loop ranks the lanes that share the first lane's digit
    // with one ballot and lets only the others issue atomics.
    const uint32_t f = digit_of(k[0]);
    const bool careful = __builtin_popcountll(__builtin_amdgcn_ballot_w64(
                             f == (uint32_t)__builtin_amdgcn_readfirstlane((int)f))) >= kWave / 4;
    if (!careful) {
#pragma unroll
      for (int i = 0; i < IPT; i++) {
        const uint32_t d = digit_of(k[i]);
        const uint32_t sh = (d & 1u) << 4;
        keep_rank(i, atomicAdd(wc + (d >> 1), 1u << sh), sh);
      }
    } else {
#pragma unroll
      for (int i = 0; i < IPT; i++) {
        const uint32_t d = digit_of(k[i]);
        const uint32_t sh = (d & 1u) << 4;
        const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
        const uint64_t same = __builtin_amdgcn_ballot_w64(d == d0);
        if (d == d0) {
          const uint32_t old = lds_load(wc + (d0 >> 1));
          const uint32_t below = __builtin_amdgcn_mbcnt_hi((uint32_t)(same >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)same, 0u));
          if (below == 0) lds_store(wc + (d0 >> 1), old + ((uint32_t)__builtin_popcountll(same) << sh));
          keep_rank(i, old + (below << sh), sh);
        } else {
          keep_rank(i, atomicAdd(wc + (d >> 1), 1u << sh), sh);
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
  __syncthreads();

  // ---- per digit (thread d): tile count, publish it, first local slot of each wave's keys
  uint32_t total = 0, lbase = 0;
  if (tid < kRadix) {
#pragma unroll
    for (int w = 0; w < NWAVES; w++) total += sm.wave_cnt[w][tid];
    const uint32_t st = (tile == 0) ? kInclusive : kPartial;
    if (tile == 0)
      for (int i = 0; i < publish_delay; i++) __builtin_amdgcn_s_sleep(127);  // test knob, 0 in normal use
    st_agent(&desc[tile * kRadix + tid], DescWord<D>::make(st, total));
    const uint32_t incl = wave_inclusive_scan(total, 0u, [](uint32_t a, uint32_t b) { return a + b; });
    if (lane == 63) sm.wave_tot[wave] = incl;
    lbase = incl - total;
  }
  __syncthreads();
  if (tid < kRadix) {
    for (int w = 0; w < wave; w++) lbase += sm.wave_tot[w];
    uint32_t run = lbase;  // counts -> first local slot of each wave's keys of this digit
#pragma unroll
    for (int w = 0; w < NWAVES; w++) {
      const uint32_t c = sm.wave_cnt[w][tid];
      sm.wave_cnt[w][tid] = (uint16_t)run;
      run += c;
    }
  }
  __syncthreads();

  // ---- reorder: local slot = first slot of the wave's keys of that digit + rank
  uint32_t pos[IPT];
#pragma unroll
  for (int i = 0; i < IPT; i++) {
    const uint32_t r = (i & 1) ? rk[i / 2] >> 16 : rk[i / 2] & 0xffffu;
    pos[i] = r + wc16[digit_of(k[i])];
    s_keys[pos[i]] = k[i];
  }

  // ---- look-back over earlier tiles (thread d for digit d), kLookW descriptors per round trip
  if (tid < kRadix) {
    uint32_t prefix = 0;
    if (tile > 0) {
      int64_t t = tile - 1;
      bool done = false;
      uint32_t spins = 0;
      while (!done) {
        D v[kLookW];
#pragma unroll
        for (int j = 0; j < kLookW; j++)
          v[j] = (t - j >= 0) ? ld_agent(&desc[(t - j) * kRadix + tid]) : DescWord<D>::make(kInclusive, 0u);
        int used = 0;
#pragma unroll
        for (int j = 0; j < kLookW; j++) {
          const uint32_t st = DescWord<D>::status(v[j]);
          if (!done && used == j && st != kInvalid) {
            prefix += DescWord<D>::count(v[j]);
            used = j + 1;
            done = st == kInclusive;
          }
        }
        t -= used;
        if (used == 0) {
          __builtin_amdgcn_s_sleep(2);
          if (++spins > spin_limit) {  // never in a working system; keeps every wait bounded
            note_timeout(status);
            done = true;
          }
        }
      }
      st_agent(&desc[tile * kRadix + tid], DescWord<D>::make(kInclusive, prefix + total));
    }
    sm.global_off[tid] = gbase[tid] + prefix - lbase;
  }
  __syncthreads();

  // ---- write each digit's run contiguously.  Full tiles (all but the last) take a path with
  //      no per-item bounds test, so the LDS reads of several items are in flight together.
  uint32_t gpos[IPT];
  auto write_keys = [&](auto full_tag) {
    constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
    for (int j = 0; j < IPT; j++) {
      const int li = j * BLOCK + tid;
      const U key = s_keys[li];
      gpos[j] = sm.global_off[digit_of(key)] + (uint32_t)li;
      if (kFull || li < valid) kout[gpos[j]] = decode_key<U, FLOAT>(key, xor_mask);
    }
  };
  if (full) write_keys(std::true_type{}); else write_keys(std::false_type{});

  if constexpr (VB > 0) {
    __syncthreads();
    auto stage_values = [&](auto full_tag) {
      constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
      for (int i = 0; i < IPT; i++) {
        const int li = slab + i * kWave;
        const V v = vin[base + (kFull || li < valid ? li : valid - 1)];  // unconditional, as for the keys
        s_vals[pos[i]] = v;
      }
    };
    if (full) stage_values(std::true_type{}); else stage_values(std::false_type{});
    __syncthreads();
    auto write_values = [&](auto full_tag) {
      constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
      for (int j = 0; j < IPT; j++) {
        const int li = j * BLOCK + tid;
        if (kFull || li < valid) vout[gpos[j]] = s_vals[li];
      }
    };
    if (full) write_values(std::true_type{}); else write_values(std::false_type{});
  }
}

// ---------------------------------------------------------------------------------------
// Inputs of up to kTileSortMax items: ONE workgroup sorts them, every pass of the LSD radix sort
// inside LDS (the shape of the reference's single-tile path, cub::DeviceRadixSortSingleTileKernel
// behind thrust/system/cuda/detail/sort.h:213-380).  No histogram pass, no descriptors, no
// alternate buffer: one launch instead of two plus one per digit, which is what a small sort
// costs.  Ranking is the onesweep kernel's: wave w owns a contiguous slab, item i of lane l is
// slab[i*64 + l], and the value returned by the wave's LDS atomic add on its counter of the key's
// digit numbers that digit's keys in (item, lane) order, the memory order: the sort is stable.
// ---------------------------------------------------------------------------------------
constexpr int kTileSortThreads = 512;
constexpr int kTileSortIpt = 8;
constexpr int kTileSortMax = kTileSortThreads * kTileSortIpt;

template <class U, int VB, bool FLOAT>
__global__ __launch_bounds__(kTileSortThreads) void tile_sort_kernel(U* keys, void* values_, int n, U xor_mask) {
  using V = typename value_of<VB>::type;
  constexpr int IPT = kTileSortIpt, BLOCK = kTileSortThreads, NW = BLOCK / kWave, P = (int)sizeof(U);
  __shared__ U s_keys[BLOCK * IPT];
  __shared__ V s_vals[VB ? BLOCK * IPT : 1];
  __shared__ uint32_t s_cnt[NW][kRadix];  // per-wave digit counts, then the first slot of each (wave, digit)
  __shared__ uint32_t s_wtot[kRadix / kWave];
  V* values = static_cast<V*>(values_);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int slab = wave * (kWave * IPT) + lane;

  U k[IPT];
  V v[IPT];
#pragma unroll
  for (int i = 0; i < IPT; i++) {  // every lane loads (a clamped index); padding sorts last and stays last
    const int li = slab + i * kWave;
    const int at = li < n ? li : n - 1;
    const U got = encode_key<U, FLOAT>(keys[at], xor_mask);
    k[i] = li < n ? got : U(~U(0));
    if (VB) v[i] = values[at];
  }

  for (int p = 0; p < P; p++) {
    const int shift = 8 * p;
    for (int j = tid; j < NW * kRadix; j += BLOCK) (&s_cnt[0][0])[j] = 0;
    __syncthreads();
    uint32_t rank[IPT];
#pragma unroll
    for (int i = 0; i < IPT; i++) rank[i] = atomicAdd(&s_cnt[wave][(uint32_t)(k[i] >> shift) & 0xffu], 1u);
    __syncthreads();
    // thread d: the digit's count per wave, the exclusive prefix over the digits, then the first
    // slot of every (wave, digit)
    uint32_t c[NW], lbase = 0;
    if (tid < kRadix) {
      uint32_t total = 0;
#pragma unroll
      for (int w = 0; w < NW; w++) {
        c[w] = s_cnt[w][tid];
        total += c[w];
      }
      const uint32_t incl = wave_inclusive_scan(total, 0u, [](uint32_t a, uint32_t b) { return a + b; });
      if (lane == kWave - 1) s_wtot[wave] = incl;
      lbase = incl - total;
    }
    __syncthreads();
    if (tid < kRadix) {
      for (int w = 0; w < wave; w++) lbase += s_wtot[w];
      uint32_t run = lbase;
#pragma unroll
      for (int w = 0; w < NW; w++) {
        s_cnt[w][tid] = run;
        run += c[w];
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < IPT; i++) {
      const uint32_t pos = s_cnt[wave][(uint32_t)(k[i] >> shift) & 0xffu] + rank[i];
      s_keys[pos] = k[i];
      if (VB) s_vals[pos] = v[i];
    }
    __syncthreads();
    // The next pass overwrites s_keys / s_vals only after three more barriers, and it uses every
    // k[i] read here as the address of its ranking atomic before the first of them: a read of
    // this pass cannot be outstanding when its source is rewritten.  (v[i] is read by the same
    // instructions' neighbours and the LDS returns a wavefront's reads in order.)
#pragma unroll
    for (int i = 0; i < IPT; i++) {
      k[i] = s_keys[slab + i * kWave];
      if (VB) v[i] = s_vals[slab + i * kWave];
    }
  }

#pragma unroll
  for (int i = 0; i < IPT; i++) {
    const int li = slab + i * kWave;
    if (li < n) {
      keys[li] = decode_key<U, FLOAT>(k[i], xor_mask);
      if (VB) values[li] = v[i];
    }
  }
}

// ---------------------------------------------------------------------------------------
// Self-test of the LDS property the ranking relies on
// ---------------------------------------------------------------------------------------
// Every wave adds 1 to pseudo-random counters of its own (uniform digits, one hot digit, and a
// bank-structured pattern) and compares each returned value with the counter's value before
// the instruction plus the number of lower lanes that hit the same counter.
__global__ __launch_bounds__(512) void lds_atomic_order_kernel(unsigned long long* mismatches, int iters) {
  __shared__ uint32_t cnt[8][kRadix];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  for (int i = threadIdx.x; i < 8 * kRadix; i += 512) (&cnt[0][0])[i] = 0;
  __syncthreads();
  unsigned long long bad = 0;
  for (int it = 0; it < iters; it++) {
    uint32_t h = (blockIdx.x * 512u + threadIdx.x) * 7919u + (uint32_t)it * 104729u + 12345u;
    h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
    const int mode = it % 3;
    const uint32_t d = mode == 0 ? (h & 0xffu) : mode == 1 ? ((h % 5u == 0) ? ((h >> 8) & 0xffu) : 3u)
                                                           : (((uint32_t)lane * 4u + (h & 3u)) & 0xffu);
    uint64_t same = ~0ull;
#pragma unroll
    for (int b = 0; b < kRadixBits; b++) {
      const bool bit = (d >> b) & 1u;
      const uint64_t m = __builtin_amdgcn_ballot_w64(bit);
      same &= bit ? m : ~m;
    }
    const uint32_t lower = (uint32_t)__builtin_popcountll(same & ((1ull << lane) - 1ull));
    const uint32_t before = lds_load(&cnt[wave][d]);
    __builtin_amdgcn_wave_barrier();
    const uint32_t got = atomicAdd(&cnt[wave][d], 1u);
    __builtin_amdgcn_wave_barrier();
    bad += got != before + lower;
  }
  if (bad) atomicAdd(mismatches, bad);
}

// The ranking's assumption is checked once per device, by the first sort that runs there: a
// short run of the kernel above on the caller's stream, whose result is waited for (the only
// time a sort call blocks).  A device that fails it gets hipErrorNotSupported from every sort
// instead of a possibly unstable result.  A call made under stream capture cannot wait and
// leaves the check to the next call that can.
__device__ unsigned long long g_order_mismatches;
constexpr int kMaxDevices = 64;
static std::atomic<int> g_order_verdict[kMaxDevices];  // 0 not checked, 1 in order, 2 not
static std::mutex g_order_mu;

static hipError_t run_lds_order_check(hipStream_t s, int iters, unsigned long long* mismatches) {
  void* sym = nullptr;
  hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_order_mismatches));
  if (e != hipSuccess) return e;
  e = zero_async(sym, sizeof(unsigned long long), s);
  if (e != hipSuccess) return e;
  // four workgroups per compute unit: every LDS unit of the device is exercised
  TCD_LAUNCH("lds_atomic_order_kernel", lds_atomic_order_kernel, dim3((unsigned)(4 * device_cu_count())), dim3(512), s,
             static_cast<unsigned long long*>(sym), iters);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  e = hipMemcpyAsync(mismatches, sym, sizeof(*mismatches), hipMemcpyDeviceToHost, s);
  if (e != hipSuccess) return e;
  return hipStreamSynchronize(s);
}

static hipError_t ensure_lds_order(hipStream_t s) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  int v = g_order_verdict[dev].load(std::memory_order_acquire);
  if (v == 1) return hipSuccess;
  if (v == 2) return hipErrorNotSupported;
  // The check blocks, so it is left to a later call when this one may be recorded into a graph.
  // A query that fails (the legacy stream while another thread captures) counts as capturing.
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cs) != hipSuccess) {
    (void)hipGetLastError();
    return hipSuccess;
  }
  if (cs != hipStreamCaptureStatusNone) return hipSuccess;
  std::lock_guard<std::mutex> g(g_order_mu);
  v = g_order_verdict[dev].load(std::memory_order_acquire);
  if (v == 0) {
    unsigned long long bad = 0;
    e = run_lds_order_check(s, 24, &bad);  // 1.2e7 checked atomics on 256 compute units
    if (e != hipSuccess) return e;
    v = bad == 0 ? 1 : 2;
    g_order_verdict[dev].store(v, std::memory_order_release);
  }
  return v == 1 ? hipSuccess : hipErrorNotSupported;
}

// ---------------------------------------------------------------------------------------
// Which form of take_tile a device gets.  The grouped form needs two things of the device:
// workgroup i runs on XCD i mod 8, and an XCD starts its next workgroup as soon as it has room,
// whether or not the other XCDs have.  Both are observed once per device by a probe whose
// workgroups wait on nothing but the clock: one workgroup per CU (they ask for 125 KiB of LDS),
// three rounds of them per XCD; those of class 0 (index 0 mod 8) stay for 60 us each, the others
// leave at once.  Every workgroup notes its XCD and when it started.  On a device of the expected
// kind the classes 1..7 are through their three rounds while class 0 is still in its first.
// Anything else — another XCD count, another partition mode, a dispatcher that serves the XCDs in
// turn — selects the plain tickets.
constexpr int kProbeMax = 4096;
__device__ unsigned long long g_probe_start[kProbeMax];
__device__ unsigned int g_probe_xcd[kProbeMax];
__global__ __launch_bounds__(1024) void xcd_dispatch_probe_kernel(unsigned long long* start, unsigned int* xcd_of, int slow_ticks) {
  __shared__ uint32_t occupy[125 * 256];  // 125 KiB: one workgroup per CU
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();  // 100 MHz
  if (threadIdx.x == 0) {
    start[blockIdx.x] = t0;
    xcd_of[blockIdx.x] = __builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15u;  // XCC_ID, bits 3:0
    occupy[blockIdx.x % (125 * 256)] = 1u;
  }
  if (blockIdx.x % kXcds == 0)
    while (__builtin_amdgcn_s_memrealtime() - t0 < (unsigned long long)slow_ticks) __builtin_amdgcn_s_sleep(32);
  if (threadIdx.x == 1 && occupy[1] == 0xdeadbeefu) start[0] = 0;  // keeps the array
}
static std::atomic<int> g_xcd_verdict[kMaxDevices];  // 0 not probed, 1 grouped tiles, 2 plain tickets
static std::atomic<int> g_force_plain_tickets{0};    // test knob
static std::mutex g_xcd_mu;

// *why: 1 the device qualifies; 0 its workgroups are not spread over 8 XCDs by index; -1 the XCDs
// were not seen to be served independently; -2 the CU count does not fit the probe
static hipError_t run_xcd_dispatch_probe(hipStream_t s, bool* grouped_ok, int* why = nullptr) {
  *grouped_ok = false;
  int why_local = 0;
  if (!why) why = &why_local;
  *why = -2;
  const int per_xcd = device_cu_count() / kXcds;
  const int wgs = kXcds * 3 * per_xcd;
  if (per_xcd < 1 || device_cu_count() % kXcds != 0 || wgs > kProbeMax) return hipSuccess;
  void *d_start = nullptr, *d_xcd = nullptr;
  hipError_t e = hipGetSymbolAddress(&d_start, HIP_SYMBOL(g_probe_start));
  if (e != hipSuccess) return e;
  e = hipGetSymbolAddress(&d_xcd, HIP_SYMBOL(g_probe_xcd));
  if (e != hipSuccess) return e;
  TCD_LAUNCH("xcd_dispatch_probe_kernel", xcd_dispatch_probe_kernel, dim3(wgs), dim3(1024), s,
             static_cast<unsigned long long*>(d_start), static_cast<unsigned int*>(d_xcd), 6000);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  std::vector<unsigned long long> start(wgs);
  std::vector<unsigned int> xcd_of(wgs);
  e = hipMemcpyAsync(start.data(), d_start, sizeof(unsigned long long) * wgs, hipMemcpyDeviceToHost, s);
  if (e != hipSuccess) return e;
  e = hipMemcpyAsync(xcd_of.data(), d_xcd, sizeof(unsigned int) * wgs, hipMemcpyDeviceToHost, s);
  if (e != hipSuccess) return e;
  e = hipStreamSynchronize(s);
  if (e != hipSuccess) return e;
  // workgroup i on XCD (i + first) mod 8, with one `first` for the whole launch: the workgroups of an
  // index class then share an XCD, which is all that the groups need
  *why = 0;
  const unsigned first = xcd_of[0];
  for (int i = 0; i < wgs; i++)
    if (xcd_of[i] >= (unsigned)kXcds || xcd_of[i] != (first + (unsigned)i) % kXcds) return hipSuccess;
  *why = -1;
  // class 0's first workgroup of the second round starts when one of its first round has left
  const unsigned long long second_round_of_slow = start[(size_t)per_xcd * kXcds];
  for (int c = 1; c < kXcds; c++)
    if (start[(size_t)(3 * per_xcd - 1) * kXcds + c] >= second_round_of_slow) return hipSuccess;  // the XCDs are not served independently
  *grouped_ok = true;
  *why = 1;
  return hipSuccess;
}

// true: the grouped form may be used by this call
static hipError_t xcd_groups_usable(hipStream_t s, bool* usable) {
  *usable = false;
  if (g_force_plain_tickets.load(std::memory_order_relaxed)) return hipSuccess;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipSuccess;
  int v = g_xcd_verdict[dev].load(std::memory_order_acquire);
  if (v == 0) {
    // the probe blocks: a later call runs it (a failing query counts as capturing, as above)
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) != hipSuccess) {
      (void)hipGetLastError();
      return hipSuccess;
    }
    if (cs != hipStreamCaptureStatusNone) return hipSuccess;
    std::lock_guard<std::mutex> g(g_xcd_mu);
    v = g_xcd_verdict[dev].load(std::memory_order_acquire);
    if (v == 0) {
      // a verdict that rests on timing (-1) is asked for up to three times before it is believed:
      // it stays for the life of the process and costs a pair sort 10 %
      bool ok = false;
      int why = 0;
      for (int attempt = 0; attempt < 3 && !ok; attempt++) {
        e = run_xcd_dispatch_probe(s, &ok, &why);
        if (e != hipSuccess) return e;
        if (why != -1) break;
      }
      v = ok ? 1 : 2;
      g_xcd_verdict[dev].store(v, std::memory_order_release);
    }
  }
  *usable = v == 1;
  return hipSuccess;
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
template <class U, int VB, bool SMALL>
struct SortConfig {
  // Tile shape by the widest element that goes through the LDS exchange buffer and by whether
  // values follow the keys, measured on MI355X at n = 2^28.  The time of a pass grows by about
  // 9 ns per tile (ticket, barriers, descriptor traffic and look-back latency do not shrink
  // with the tile) and longer per-digit runs write fuller cache lines, so tiles are as large as
  // LDS and registers allow: one 1024-thread workgroup per CU with up to 128 VGPRs and
  // 120-155 KiB of LDS (32768 keys of up to 4 bytes, with or without values; 18432 wider ones).
  static constexpr int ELEM = (int)sizeof(U) > VB ? (int)sizeof(U) : VB;
  static constexpr int CLASS = ELEM <= 4 ? (VB == 0 ? 0 : 1) : (VB == 0 ? 2 : 3);  // A, P, B, C
  // Inputs too small to give every CU a few of those tiles use 512 x 16 tiles instead.
  static constexpr int BLOCK = SMALL ? 512 : 1024;
  static constexpr int IPT = SMALL ? 16 : (CLASS <= 1 ? 32 : 18);
  static constexpr int TILE = BLOCK * IPT;
  // wavefronts per SIMD the register allocation aims for
  static constexpr int WPE = 4;
};
// Below this many items the small tiles are faster (measured crossover: 2^21 keys, 2^22 pairs).
// positions, digit counts and their prefix sums are 32-bit
constexpr int64_t kSortMaxN = (int64_t(1) << 32) - 1;
constexpr int64_t small_sort_limit(int value_bytes) { return int64_t(1) << (21 + (value_bytes ? 1 : 0)); }

struct SortPlan {
  size_t status, keys_alt, vals_alt, hist, tickets, xcd, desc, total;
  int xcd_slots;  // groups an XCD may take in one pass
  size_t zero_begin, zero_bytes;  // cleared by a launch of its own before anything else
  size_t desc_bytes;              // cleared by the histogram kernel
  int64_t ntiles;
};

// One-byte keys without values are not moved at all: their sorted sequence is the 256 runs that the
// histogram describes.  Thread t writes 16 output bytes at a time; the digit of its first byte is
// found by bisection over the 256 run starts, and nearly every 16-byte piece lies inside one run.
constexpr int kFillThreads = 256;
__global__ __launch_bounds__(kFillThreads) void counting_fill_kernel(uint8_t* out, int64_t n, uint8_t xor_mask,
                                                                   const uint32_t* __restrict__ gbase) {
  __shared__ uint32_t s_start[kRadix + 1];
  s_start[threadIdx.x] = gbase[threadIdx.x];
  if (threadIdx.x == 0) s_start[kRadix] = (uint32_t)n;  // n < 2^32 - 1
  __syncthreads();
  const int64_t pieces = (n + 15) / 16;
  for (int64_t c = (int64_t)blockIdx.x * kFillThreads + threadIdx.x; c < pieces; c += (int64_t)gridDim.x * kFillThreads) {
    const int64_t p0 = c * 16;
    int d = 0;  // the last digit whose run starts at or before p0 (empty runs before it share its start)
#pragma unroll
    for (int step = kRadix / 2; step > 0; step >>= 1)
      if ((int64_t)s_start[d + step] <= p0) d += step;
    if ((int64_t)s_start[d + 1] >= p0 + 16) {  // one run covers the piece (and the piece lies inside the output)
      const uint32_t w = (uint32_t)(uint8_t)(d ^ xor_mask) * 0x01010101u;
      tcd_v4u v;
      v.x = v.y = v.z = v.w = w;
      store16(out + p0, v);
    } else {
      const int count = (int)(n - p0 < 16 ? n - p0 : 16);
#pragma unroll 1
      for (int j = 0; j < count; j++) {
        while ((int64_t)s_start[d + 1] <= p0 + j) d++;  // ends: s_start[256] = n > p0 + j
        out[p0 + j] = (uint8_t)(d ^ xor_mask);
      }
    }
  }
}

constexpr int kHistDoneWord = 8;  // in the 64 words of the ticket block
constexpr size_t kSortStatusOffset = 0;  // of the status word in a sort call's temporary storage
static std::atomic<uint32_t> g_test_spin_limit{kLookbackSpinLimit};  // test knob
static constexpr size_t xcd_words_per_pass(int slots) { return (size_t)kXcds * kXcdCounterStride + (size_t)kXcds * (size_t)slots; }
template <class U, int VB, class C, class D>
static SortPlan make_plan(int64_t n) {
  constexpr int P = sizeof(U);
  SortPlan p{};
  p.ntiles = ceil_div(n, C::TILE);
  size_t off = 0;
  constexpr bool kCounting = sizeof(U) == 1 && VB == 0;  // histogram and fill: no alternate buffer, no descriptors
  // what starts at zero comes first; its first word is the call's status (kSortStatusOffset)
  p.zero_begin = off;
  p.status = off; off += 256;
  p.hist = off; off += align_up((size_t)P * kRadix * 4, 256);
  p.tickets = off; off += 256;  // a counter per pass (at most 8), and the histogram kernel's count of finished workgroups
  // per pass: a counter per XCD (a cache line each) and the numbers of the groups each XCD took
  p.xcd_slots = (int)ceil_div(p.ntiles, (int64_t)kXcds * kXcdGroup);
  p.xcd = off; off += kCounting ? 0 : align_up((size_t)P * xcd_words_per_pass(p.xcd_slots) * 4, 256);
  p.zero_bytes = off - p.zero_begin;
  // the descriptors start at zero too: the histogram kernel clears them
  p.desc = off; off += kCounting ? 0 : align_up((size_t)P * p.ntiles * kRadix * sizeof(D), 256);
  p.desc_bytes = off - p.desc;
  p.keys_alt = off; off += kCounting ? 0 : align_up((size_t)n * sizeof(U), 256);
  p.vals_alt = off; off += align_up((size_t)n * VB, 256);
  p.total = off;
  return p;
}

template <class U, int VB, bool FLOAT, class C, class D>
static hipError_t sort_with(void* temp, size_t* temp_bytes, void* keys, void* values, int64_t n,
                            U xor_mask, hipStream_t stream) {
  constexpr int P = sizeof(U);
  const SortPlan plan = make_plan<U, VB, C, D>(n);
  if (temp == nullptr) {
    *temp_bytes = plan.total;
    return hipSuccess;
  }
  if (*temp_bytes < plan.total) return hipErrorInvalidValue;
  if (n == 0) return hipSuccess;
  {
    const hipError_t oe = ensure_lds_order(stream);
    if (oe != hipSuccess) return oe;
  }
  if (n <= kTileSortMax) {  // one workgroup, one launch, nothing of `temp` is used
    TCD_LAUNCH("tile_sort_kernel", (tile_sort_kernel<U, VB, FLOAT>), dim3(1), dim3(kTileSortThreads), stream,
               static_cast<U*>(keys), values, (int)n, xor_mask);
    return hipGetLastError();
  }
  char* t = static_cast<char*>(temp);
  U* kbuf[2] = {static_cast<U*>(keys), reinterpret_cast<U*>(t + plan.keys_alt)};
  char* vbuf[2] = {static_cast<char*>(values), t + plan.vals_alt};
  uint32_t* ghist = reinterpret_cast<uint32_t*>(t + plan.hist);
  uint32_t* tickets = reinterpret_cast<uint32_t*>(t + plan.tickets);
  D* desc = reinterpret_cast<D*>(t + plan.desc);
  static_assert(kSortStatusOffset == 0, "thrust_cdna4_sort_status reads the first word");
  uint32_t* status = reinterpret_cast<uint32_t*>(t + plan.status);
  const uint32_t spin_limit = g_test_spin_limit.load(std::memory_order_relaxed);
  const int publish_delay = lookback_test_publish_delay();

  hipError_t e = zero_async(t + plan.zero_begin, plan.zero_bytes, stream);
  if (e != hipSuccess) return e;

  // passes over places where all keys agree are skipped on the device; with an even number of
  // places the passes that run are an even number too and the result ends in the caller's buffer
  constexpr int kSkipping = (P % 2 == 0) ? 1 : 0;
  const int vec_ok = (reinterpret_cast<uintptr_t>(keys) & (sizeof(U) - 1)) == 0;  // see load16
  int64_t hblocks = ceil_div(n, kHistThreads * 64);
  const int cus = device_cu_count();
  if (hblocks > cus) hblocks = cus;  // one workgroup per CU, eight loads in flight per thread: 1 % of a 2^28 sort over two with two
  TCD_LAUNCH("radix_hist_kernel", (radix_hist_kernel<U, FLOAT>), dim3((unsigned)hblocks), dim3(kHistThreads), stream,
             kbuf[0], n, xor_mask, ghist, vec_ok, static_cast<void*>(t + plan.desc), plan.desc_bytes,
             tickets, tickets + kHistDoneWord, kSkipping);
  if constexpr (sizeof(U) == 1 && VB == 0) {
    int64_t fblocks = ceil_div(n, (int64_t)kFillThreads * 16 * 4);
    if (fblocks > (int64_t)cus * 8) fblocks = (int64_t)cus * 8;
    TCD_LAUNCH("counting_fill_kernel", counting_fill_kernel, dim3((unsigned)fblocks), dim3(kFillThreads), stream,
               reinterpret_cast<uint8_t*>(kbuf[0]), n, (uint8_t)xor_mask, ghist);
    return hipGetLastError();
  }
  // tiles in groups per XCD where the device was seen to allow it and every XCD has several groups to
  // take; the grid is then padded so that each XCD's share of the workgroups is whole groups
  bool grouped = false;
  if (plan.ntiles >= (int64_t)kXcds * kXcdGroup * 4) {
    e = xcd_groups_usable(stream, &grouped);
    if (e != hipSuccess) return e;
  }
  const int64_t grid = grouped ? (int64_t)kXcds * kXcdGroup * plan.xcd_slots : plan.ntiles;
  for (int p = 0; p < P; p++) {
    uint32_t* xcd = grouped ? reinterpret_cast<uint32_t*>(t + plan.xcd) + (size_t)p * xcd_words_per_pass(plan.xcd_slots) : nullptr;
    TCD_LAUNCH("onesweep_kernel", (onesweep_kernel<U, VB, FLOAT, C::BLOCK, C::IPT, C::WPE, D>), dim3((unsigned)grid),
               dim3(C::BLOCK), stream, kbuf[0], kbuf[1], static_cast<void*>(vbuf[0]), static_cast<void*>(vbuf[1]), n, xor_mask, 8 * p,
               ghist + p * kRadix, desc + (size_t)p * plan.ntiles * kRadix, tickets + p, xcd, plan.xcd_slots,
               status, spin_limit, publish_delay);
  }
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (P % 2 == 1) {  // an odd number of passes, none skipped: bring the result home
    e = copy_async(kbuf[0], kbuf[1], (size_t)n * sizeof(U), stream);
    if (e != hipSuccess) return e;
    if (VB) e = copy_async(vbuf[0], vbuf[1], (size_t)n * VB, stream);
  }
  return e;
}

template <class U, int VB, bool FLOAT>
static hipError_t sort_typed(void* temp, size_t* temp_bytes, void* keys, void* values, int64_t n,
                             U xor_mask, hipStream_t stream) {
  // the choice depends on n only, so the size query and the run agree
  if (n < small_sort_limit(VB))
    return sort_with<U, VB, FLOAT, SortConfig<U, VB, true>, uint32_t>(temp, temp_bytes, keys, values, n, xor_mask, stream);
  if (n < (int64_t(1) << 30))  // counts fit the 30 bits of a 32-bit descriptor word
    return sort_with<U, VB, FLOAT, SortConfig<U, VB, false>, uint32_t>(temp, temp_bytes, keys, values, n, xor_mask, stream);
  return sort_with<U, VB, FLOAT, SortConfig<U, VB, false>, uint64_t>(temp, temp_bytes, keys, values, n, xor_mask, stream);
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
  if (!temp_bytes || n < 0 || n >= tcd::kSortMaxN || tcd::temp_misaligned(temp) || (n > 0 && temp && !keys))
    return hipErrorInvalidValue;
  return (int)tcd::sort_dispatch<0>(temp, temp_bytes, key_dtype, keys, nullptr, n, descending,
                                    static_cast<hipStream_t>(stream));
}

extern "C" int thrust_cdna4_sort_pairs(void* temp, size_t* temp_bytes, int key_dtype, void* keys,
                                       int value_bytes, void* values, int64_t n, int descending,
                                       void* stream) {
  if (!temp_bytes || n < 0 || n >= tcd::kSortMaxN || tcd::temp_misaligned(temp) || (n > 0 && temp && (!keys || !values)))
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

extern "C" int thrust_cdna4_set_test_sort_plain_tickets(int on) {
  return tcd::g_force_plain_tickets.exchange(on ? 1 : 0);
}

extern "C" int thrust_cdna4_selftest_xcd_dispatch(int* grouped, void* stream) {
  if (!grouped) return hipErrorInvalidValue;
  bool ok = false;
  int why = 0;
  std::lock_guard<std::mutex> g(tcd::g_xcd_mu);  // the probe's device arrays have one user at a time
  const hipError_t e = tcd::run_xcd_dispatch_probe(static_cast<hipStream_t>(stream), &ok, &why);
  *grouped = why;
  return (int)e;
}

extern "C" int thrust_cdna4_sort_tile_assignment(int* form) {
  if (!form) return hipErrorInvalidValue;
  int dev = 0;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  *form = (dev >= 0 && dev < tcd::kMaxDevices) ? tcd::g_xcd_verdict[dev].load(std::memory_order_acquire) : 2;
  return hipSuccess;
}

extern "C" int thrust_cdna4_set_test_sort_spin_limit(long long polls) {
  const uint32_t v = polls < 0 ? tcd::kLookbackSpinLimit : (uint32_t)(polls > 0xffffffffLL ? 0xffffffffLL : polls);
  return (int)tcd::g_test_spin_limit.exchange(v, std::memory_order_relaxed);
}

extern "C" int thrust_cdna4_sort_status(const void* temp, int64_t n, void* stream) {
  using namespace tcd;
  if (n < 0 || (n > kTileSortMax && !temp)) return hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e;
  uint32_t word = 0;
  if (n > kTileSortMax) {  // smaller sorts are one workgroup: no look-back, and nothing of `temp` is used
    e = hipMemcpyAsync(&word, static_cast<const char*>(temp) + kSortStatusOffset, sizeof(word), hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return (int)e;
  }
  e = hipStreamSynchronize(s);
  if (e != hipSuccess) return (int)e;
  if (word == 0) return hipSuccess;
  // a wait that did not end: whatever the reason, later sorts on this device hand their tiles
  // out from the single counter, whose waits depend on nothing the probe had to observe
  int dev = 0;
  if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices) g_xcd_verdict[dev].store(2, std::memory_order_release);
  return hipErrorLaunchTimeOut;
}

extern "C" int thrust_cdna4_lookback_timeout_counter(void** device_address) {
  if (!device_address) return hipErrorInvalidValue;
  return (int)hipGetSymbolAddress(device_address, HIP_SYMBOL(tcd::g_lookback_timeouts));
}

extern "C" int thrust_cdna4_lookback_timeouts(unsigned long long* count) {
  if (!count) return hipErrorInvalidValue;
  unsigned int c = 0;
  const hipError_t e = hipMemcpyFromSymbol(&c, HIP_SYMBOL(tcd::g_lookback_timeouts), sizeof(c));
  *count = c;
  return (int)e;
}

extern "C" int thrust_cdna4_selftest_lds_atomic_order(long long* mismatches, void* stream) {
  using namespace tcd;
  if (!mismatches) return hipErrorInvalidValue;
  unsigned long long bad = 0;
  std::lock_guard<std::mutex> g(g_order_mu);  // one user of the result word at a time
  const hipError_t e = run_lds_order_check(static_cast<hipStream_t>(stream), 600, &bad);
  *mismatches = (long long)bad;
  return (int)e;
}
